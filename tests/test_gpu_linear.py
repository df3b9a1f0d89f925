"""Fused linear kernel (C-ABI spgt_linear_forward) against a float64 CPU product.

The expected values are a plain float64 matmul + bias + activation + residual, the
definition of nn.Linear followed by the elementwise steps of network/layer.py:155-174;
tolerance 1e-5 of the output scale (fp32 accumulation over at most 256 terms).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _expected(x, w_kn, b, act, res, after):
    y = x.double() @ w_kn.double()
    if b is not None:
        y = y + b.double()
    if res is not None and not after:
        y = y + res.double()
    if act == "relu":
        y = torch.relu(y)
    elif act == "silu":
        y = y * torch.sigmoid(y)
    if res is not None and after:
        y = y + res.double()
    return y


@pytest.mark.parametrize("K,N", [(128, 128), (128, 256), (128, 384), (256, 128), (136, 128), (64, 64), (64, 256),
                                 (128, 64), (64, 32), (128, 96)])
@pytest.mark.parametrize("T", [1, 31, 1000, 20164])
def test_linear_shapes(gpu, K, N, T):
    from spgt_amd.extension.bind.linear import fused_linear, linear_supported
    assert linear_supported(K, N)
    g = torch.Generator().manual_seed(K * 1000 + N + T)
    x = torch.randn(T, K, generator=g)
    w = torch.randn(K, N, generator=g) / K ** 0.5
    b = torch.randn(N, generator=g)
    got = fused_linear(x.to(gpu), w.to(gpu), b.to(gpu)).cpu()
    want = _expected(x, w, b, "none", None, False)
    assert got.shape == (T, N)
    assert (got.double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("act", ["none", "relu", "silu"])
@pytest.mark.parametrize("res_mode", [None, "before", "after"])
@pytest.mark.parametrize("use_bias", [True, False])
def test_linear_epilogues(gpu, act, res_mode, use_bias):
    from spgt_amd.extension.bind.linear import fused_linear
    T, K, N = 777, 128, 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 259, K, generator=g)  # leading dims are flattened
    w = torch.randn(K, N, generator=g) / K ** 0.5
    b = torch.randn(N, generator=g) if use_bias else None
    res = torch.randn(3, 259, N, generator=g) if res_mode else None
    got = fused_linear(x.to(gpu), w.to(gpu), b.to(gpu) if use_bias else None, act,
                       res.to(gpu) if res_mode else None, res_mode == "after").cpu()
    want = _expected(x, w, b, act, res, res_mode == "after")
    assert got.shape == (3, 259, N)
    assert (got.double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


def test_linear_strided_rows(gpu):
    """x taken as a column slice of a packed [T, 384] tensor (row stride 384)."""
    from spgt_amd.extension.bind.linear import fused_linear
    g = torch.Generator().manual_seed(9)
    packed = torch.randn(500, 384, generator=g)
    w = torch.randn(128, 128, generator=g) / 128 ** 0.5
    pd = packed.to(gpu)
    got = fused_linear(pd[:, 128:256], w.to(gpu)).cpu()
    want = packed[:, 128:256].double() @ w.double()
    assert (got.double() - want).abs().max().item() <= 1e-5 * want.abs().max().item()


def test_linear_output_planes(gpu):
    """planes=3: the packed projection's column thirds come back as three contiguous tensors."""
    from spgt_amd.extension.bind.linear import fused_linear
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 333, 128, generator=g)
    w = torch.randn(128, 384, generator=g) / 128 ** 0.5
    b = torch.randn(384, generator=g)
    got = fused_linear(x.to(gpu), w.to(gpu), b.to(gpu), planes=3)
    assert got.shape == (3, 2, 333, 128) and got.is_contiguous()
    want = (x.double() @ w.double() + b.double()).view(2, 333, 3, 128).permute(2, 0, 1, 3)
    assert (got.cpu().double() - want).abs().max().item() <= 1e-5 * want.abs().max().item()
    with pytest.raises(ValueError):
        fused_linear(x.to(gpu), w.to(gpu), b.to(gpu), planes=5)


@pytest.mark.parametrize("K,N,planes", [(64, 128, 1), (128, 128, 1), (128, 384, 3), (136, 128, 1), (256, 128, 1),
                                        (256, 256, 1)])
@pytest.mark.parametrize("act,res_mode", [("none", None), ("silu", None), ("relu", "before"), ("none", "after")])
def test_linear_long_inputs(gpu, K, N, planes, act, res_mode):
    """70001 tokens (a ragged last tile): the size class that runs on role-split workgroups, one per CU.
    Expected values from a float64 product on the GPU (the CPU product of this size takes too long)."""
    from spgt_amd.extension.bind.linear import fused_linear
    T = 70001
    g = torch.Generator().manual_seed(K + N)
    wide = torch.randn(T, K + 4, generator=g).to(gpu)
    x = wide[:, 4:] if K % 8 == 0 else wide[:, :K].contiguous()  # a strided view where K allows the alignment
    w = (torch.randn(K, N, generator=g) / K ** 0.5).to(gpu)
    b = torch.randn(N, generator=g).to(gpu)
    res = torch.randn(T, N, generator=g).to(gpu) if res_mode and planes == 1 else None
    got = fused_linear(x, w, b, act, res, res_mode == "after", planes=planes)
    want = _expected(x, w, b, act, res, res_mode == "after")
    if planes > 1:
        assert got.shape == (planes, T, N // planes)
        got = got.permute(1, 0, 2).reshape(T, N)
    err = (got.double() - want).abs().max().item()
    assert err <= 1e-5 * max(1.0, want.abs().max().item())
    # nothing written past the last row's neighbours: the rows around the ragged end are exact too
    assert torch.isfinite(got[-70:]).all()


@pytest.mark.parametrize("E", [1, 2, 4])
def test_linear_extra_columns(gpu, E):
    """x_extra @ weight_extra_kn added in the epilogue equals a Linear over the concatenated input
    (network/sp_model.py:59-60 concatenates the grid coordinates)."""
    from spgt_amd.extension.bind.linear import fused_linear
    g = torch.Generator().manual_seed(21 + E)
    x = torch.randn(3, 211, 128, generator=g)
    xe = torch.randn(3, 211, E, generator=g)
    w = torch.randn(128 + E, 64, generator=g) / 11.0
    b = torch.randn(64, generator=g)
    want = _expected(torch.cat([x, xe], -1), w, b, "silu", None, False)
    got = fused_linear(x.to(gpu), w[:128].contiguous().to(gpu), b.to(gpu), "silu", x_extra=xe.to(gpu),
                       weight_extra_kn=w[128:].contiguous().to(gpu)).cpu()
    assert (got.double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


def test_linear_matches_nn_linear(gpu):
    """Same result as torch's own Linear on the device, to fp32 rounding."""
    from spgt_amd.extension.bind.linear import fused_linear
    torch.manual_seed(3)
    lin = torch.nn.Linear(136, 128).to(gpu)
    x = torch.randn(4, 1001, 136, device=gpu)
    with torch.no_grad():
        want = torch.nn.functional.silu(lin(x))
        got = fused_linear(x, lin.weight.t().contiguous(), lin.bias, "silu")
    assert (got - want).abs().max().item() <= 1e-5 * want.abs().max().item()


def test_linear_errors(gpu):
    from spgt_amd._lib import SpgtError
    from spgt_amd.extension.bind.linear import fused_linear, linear_supported
    assert not linear_supported(100, 128)
    assert not linear_supported(128, 1)
    x = torch.randn(8, 100, device=gpu)
    w = torch.randn(100, 128, device=gpu)
    with pytest.raises(SpgtError):
        fused_linear(x, w)
    with pytest.raises(ValueError):
        fused_linear(torch.randn(8, 128, device=gpu), torch.randn(128, 128, device=gpu), activation="tanh")
    with pytest.raises(SpgtError):
        fused_linear(torch.randn(8, 128), torch.randn(128, 128, device=gpu))
    out = fused_linear(torch.empty(0, 128, device=gpu), torch.randn(128, 128, device=gpu))
    assert out.shape == (0, 128)


@pytest.mark.parametrize("K,HID", [(64, 256), (64, 128), (128, 256), (128, 128), (32, 128), (32, 256)])
@pytest.mark.parametrize("T", [1, 45, 5000])
@pytest.mark.parametrize("act", ["relu", "silu"])
def test_ffn_scalar(gpu, K, HID, T, act):
    """Both FeedForward layers with one output feature in one kernel, against float64."""
    from spgt_amd.extension.bind.linear import ffn_scalar_supported, fused_ffn_scalar
    assert ffn_scalar_supported(K, HID) and not ffn_scalar_supported(96, 256)
    g = torch.Generator().manual_seed(K + HID + T)
    x = torch.randn(T, K, generator=g)
    w1 = torch.randn(K, HID, generator=g) / K ** 0.5
    b1 = torch.randn(HID, generator=g)
    w2 = torch.randn(1, HID, generator=g) / HID ** 0.5
    b2 = torch.randn(1, generator=g)
    got = fused_ffn_scalar(x.to(gpu), w1.to(gpu), b1.to(gpu), w2.to(gpu), b2.to(gpu), act).cpu()
    h = _expected(x, w1, b1, act, None, False)
    want = h @ w2.double().t() + b2.double()
    assert got.shape == (T, 1)
    assert (got.double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


def test_feedforward_module_scalar_head(gpu):
    """FeedForward(64 -> 256 -> 1) under no_grad takes the one-kernel path and matches its nn.Linear graph."""
    from spgt_amd.network.layer import FeedForward
    torch.manual_seed(2)
    ffn = FeedForward(64, 1, 256, 0.0, "silu").to(gpu)
    x = torch.randn(2, 37, 37, 64, device=gpu)
    want = ffn.layer2(ffn.activation_layer(ffn.layer1(x))).detach()
    with torch.no_grad():
        got = ffn(x)
    assert got.shape == want.shape
    assert (got - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("K1", [128, 136])
@pytest.mark.parametrize("T", [1, 33, 5041])
@pytest.mark.parametrize("act", ["relu", "silu"])
def test_encoder_tail(gpu, K1, T, act):
    """fc_layer + residual + FeedForward + residual (network/sp_layer.py:75, 97-103; network/layer.py:155-174)
    in one kernel, against the same chain in float64."""
    from spgt_amd.extension.bind.linear import encoder_tail_supported, fused_encoder_tail
    assert encoder_tail_supported(K1, 128, 256) and not encoder_tail_supported(K1, 128, 512)
    g = torch.Generator().manual_seed(K1 + T)
    a = torch.randn(T, K1, generator=g)
    x = torch.randn(T, 128, generator=g)
    wfc, bfc = torch.randn(K1, 128, generator=g) / K1 ** 0.5, torch.randn(128, generator=g)
    w1, b1 = torch.randn(128, 256, generator=g) / 128 ** 0.5, torch.randn(256, generator=g)
    w2, b2 = torch.randn(256, 128, generator=g) / 16.0, torch.randn(128, generator=g)
    got = fused_encoder_tail(*[v.to(gpu) for v in (a, x, wfc, bfc, w1, b1, w2, b2)], act).cpu().double()
    y1 = x.double() + a.double() @ wfc.double() + bfc.double()
    want = y1 + _expected(y1, w1, b1, act, None, False) @ w2.double() + b2.double()
    assert got.shape == want.shape
    assert (got - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item())

@pytest.mark.parametrize("variant", ["plain136", "plain128", "folded"])
def test_encoder_tail_dropout(gpu, variant):
    """The tail's two dropouts (the reference's always-on F.dropout of fc_layer's and of the feed-forward net's
    output, network/sp_layer.py:76 and network/layer.py:173).  The masks are the library's own, so the test is of
    their properties: every element of the dropped term is either 0 or the undropped value / (1 - p); the kept
    fraction is 1 - p overall, per column and per token; neighbouring columns, neighbouring tokens and the two sites
    are uncorrelated; one seed repeats, another differs; rate 0 is the kernel without dropout, bit for bit."""
    from spgt_amd.extension.bind.linear import fused_encoder_tail, fused_encoder_tail_folded
    g = torch.Generator().manual_seed(11)
    B, S = 3, 3333
    T, p = B * S, 0.3
    K1 = 136 if variant == "plain136" else 128
    x = torch.randn(B, S, 128, generator=g).to(gpu)
    bfc = torch.randn(128, generator=g).to(gpu)
    w1, b1 = (torch.randn(128, 256, generator=g) / 128 ** 0.5).to(gpu), torch.randn(256, generator=g).to(gpu)
    w2, b2 = (torch.randn(256, 128, generator=g) / 16.0).to(gpu), torch.randn(128, generator=g).to(gpu)
    if variant == "folded":
        q = torch.randn(B, S, 128, generator=g).to(gpu)
        pos = torch.rand(B, S, 2, generator=g).to(gpu)
        ffc = (torch.randn(B, 128, 128, generator=g) / 11.0).to(gpu)
        fpos = torch.randn(B, 2, 128, generator=g).to(gpu)
        run = lambda w2_, b2_, **kw: fused_encoder_tail_folded(q, pos, x, ffc, fpos, bfc, w1, b1, w2_, b2_, "silu", **kw)
    else:
        a = torch.randn(B, S, K1, generator=g).to(gpu)
        wfc = (torch.randn(K1, 128, generator=g) / K1 ** 0.5).to(gpu)
        run = lambda w2_, b2_, **kw: fused_encoder_tail(a, x, wfc, bfc, w1, b1, w2_, b2_, "silu", **kw)
    z2, zb = torch.zeros_like(w2), torch.zeros_like(b2)
    seed = torch.tensor([12345, 678], dtype=torch.int32, device=gpu)
    seed2 = torch.tensor([12346, 678], dtype=torch.int32, device=gpu)
    y1 = run(z2, zb)                     # x + fc
    full = run(w2, b2)                   # y1 + ffn
    assert torch.equal(run(w2, b2, fc_droprate=0.0, ffn_droprate=0.0, seed=seed), full)

    def check_site(dropped, base, term, what):
        """dropped = base + mask * term / (1 - p); returns the mask [T, 128]."""
        d = (dropped - base).reshape(T, 128).double()
        t = term.reshape(T, 128).double() / (1 - p)
        tol = 2e-5 * max(1.0, t.abs().max().item())
        # (the kernel with dropout adds the residual after the position rows, the one without before them: `base`
        # may differ from the kernel's own value in the last bit, so "dropped" is |d| < tol rather than d == 0)
        keep = d.abs() > 0.5 * t.abs()
        clear = t.abs() > 10 * tol          # elements whose term tells the two cases apart: all but a handful
        assert clear.float().mean().item() > 0.995, what
        assert ((d - t).abs()[keep & clear] < tol).all(), what
        assert (d.abs()[~keep & clear] < tol).all(), what
        keep = keep | ~clear                # (counted as kept: at most 0.5 % of the elements)
        frac = keep.float().mean().item()
        assert frac == pytest.approx(1 - p, abs=3e-3), what
        assert (keep.float().mean(0) - (1 - p)).abs().max().item() < 0.03, what            # per column, 10k tokens
        per_token = keep.float().mean(1)
        assert per_token.std().item() == pytest.approx((p * (1 - p) / 128) ** 0.5, rel=0.1), what
        assert (keep[:, 1:] & keep[:, :-1]).float().mean().item() == pytest.approx((1 - p) ** 2, abs=4e-3), what
        assert (keep[1:] & keep[:-1]).float().mean().item() == pytest.approx((1 - p) ** 2, abs=4e-3), what
        return keep

    # the fc site alone (feed-forward weights zero: out = y1)
    d_fc = run(z2, zb, fc_droprate=p, seed=seed)
    m_fc = check_site(d_fc, x, y1 - x, "fc site")
    assert torch.equal(d_fc, run(z2, zb, fc_droprate=p, seed=seed))
    m_other = check_site(run(z2, zb, fc_droprate=p, seed=seed2), x, y1 - x, "fc site, another seed")
    assert (m_fc != m_other).float().mean().item() == pytest.approx(2 * p * (1 - p), abs=5e-3)
    # the feed-forward site alone
    d_ffn = run(w2, b2, ffn_droprate=p, seed=seed)
    m_ffn = check_site(d_ffn, y1, full - y1, "ffn site")
    assert (m_fc & m_ffn).float().mean().item() == pytest.approx((1 - p) ** 2, abs=4e-3)
    # both: a seed is drawn when none is given, and two calls differ
    o1, o2 = run(w2, b2, fc_droprate=p, ffn_droprate=p), run(w2, b2, fc_droprate=p, ffn_droprate=p)
    assert not torch.equal(o1, o2) and torch.isfinite(o1).all()
    torch.manual_seed(5)
    o3 = run(w2, b2, fc_droprate=p, ffn_droprate=p)
    torch.manual_seed(5)
    assert torch.equal(o3, run(w2, b2, fc_droprate=p, ffn_droprate=p))
    with pytest.raises(Exception):
        run(w2, b2, fc_droprate=1.0)


@pytest.mark.parametrize("K1", [128, 136])
@pytest.mark.parametrize("T", [8192 + 5, 70001])
def test_encoder_tail_many_tiles(gpu, K1, T):
    """More 32-token tiles than compute units, so that workgroups loop (a tile in LDS, the next one's rows in
    flight) and some take one tile more than others; a ragged last tile.  Expected values in float64 on the GPU.
    The attention rows are a strided view (row stride K1 + 8)."""
    from spgt_amd.extension.bind.linear import fused_encoder_tail
    g = torch.Generator().manual_seed(K1 * 7 + T)
    wide = torch.randn(T, K1 + 8, generator=g).to(gpu)
    a = wide[:, 8:]
    x = torch.randn(T, 128, generator=g).to(gpu)
    wfc, bfc = (torch.randn(K1, 128, generator=g) / K1 ** 0.5).to(gpu), torch.randn(128, generator=g).to(gpu)
    w1, b1 = (torch.randn(128, 256, generator=g) / 128 ** 0.5).to(gpu), torch.randn(256, generator=g).to(gpu)
    w2, b2 = (torch.randn(256, 128, generator=g) / 16.0).to(gpu), torch.randn(128, generator=g).to(gpu)
    got = fused_encoder_tail(a, x, wfc, bfc, w1, b1, w2, b2, "silu").double()
    y1 = x.double() + a.double() @ wfc.double() + bfc.double()
    want = y1 + _expected(y1, w1, b1, "silu", None, False) @ w2.double() + b2.double()
    assert (got - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item())
    # a second call on the same inputs gives the same bits (fixed summation order, no atomics)
    again = fused_encoder_tail(a, x, wfc, bfc, w1, b1, w2, b2, "silu").double()
    assert torch.equal(got, again)

@pytest.mark.parametrize("act", ["none", "relu", "silu"])
def test_linear_long_inputs_wide_output_without_planes_or_bias(gpu, act):
    """128 -> 384 on 70001 tokens into one [T, 384] tensor, no bias: the resident-weight kernel's other output
    form (the packed projection above writes three planes)."""
    from spgt_amd.extension.bind.linear import fused_linear
    T = 70001
    g = torch.Generator().manual_seed(384)
    x = torch.randn(T, 128, generator=g).to(gpu)
    w = (torch.randn(128, 384, generator=g) / 128 ** 0.5).to(gpu)
    got = fused_linear(x, w, None, act)
    want = _expected(x, w, None, act, None, False)
    assert got.shape == (T, 384)
    assert (got.double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())
    assert torch.equal(got, fused_linear(x, w, None, act))


def test_hand_written_mfma_statements_match_the_compilers_intrinsic(gpu):
    """linear_resident_k and encoder_tail_k issue their MFMAs as assembly statements with hand-counted wait states,
    which the compiler's hazard recognizer does not see.  The build makes a second library in which the same
    helpers are the compiler's intrinsic; the two must agree bit for bit on the kernels that use them (same
    instruction, same operands, same order), so a toolchain change that breaks the hand-written form fails here."""
    import os
    from spgt_amd import _lib, build
    from spgt_amd.extension.bind.linear import fused_encoder_tail, fused_encoder_tail_folded, fused_linear
    assert os.path.exists(build.CHECK_LIB_PATH), "build the library with `python -m spgt_amd.build`"
    main, check = _lib.load(), _lib.open_library(build.CHECK_LIB_PATH)

    def on(lib, fn):
        _lib._lib = lib
        try:
            return fn()
        finally:
            _lib._lib = main

    g = torch.Generator().manual_seed(2024)
    T = 70001
    x = torch.randn(T, 128, generator=g).to(gpu)
    w = (torch.randn(128, 384, generator=g) / 128 ** 0.5).to(gpu)
    b = torch.randn(384, generator=g).to(gpu)
    for act in ("none", "silu"):
        for planes in (1, 3):
            call = lambda: fused_linear(x, w, b, act, planes=planes)  # 128 -> 384 on a long input: linear_resident_k
            assert torch.equal(on(main, call), on(check, call))
    for K1 in (128, 136):
        a = torch.randn(T, K1, generator=g).to(gpu)
        wfc, bfc = (torch.randn(K1, 128, generator=g) / K1 ** 0.5).to(gpu), torch.randn(128, generator=g).to(gpu)
        w1, b1 = (torch.randn(128, 256, generator=g) / 128 ** 0.5).to(gpu), torch.randn(256, generator=g).to(gpu)
        w2, b2 = (torch.randn(256, 128, generator=g) / 16.0).to(gpu), torch.randn(128, generator=g).to(gpu)
        call = lambda: fused_encoder_tail(a, x, wfc, bfc, w1, b1, w2, b2, "silu")
        assert torch.equal(on(main, call), on(check, call))
    B, S = 3, 23333
    q, xr = torch.randn(B, S, 128, generator=g).to(gpu), torch.randn(B, S, 128, generator=g).to(gpu)
    pos = torch.rand(B, S, 2, generator=g).to(gpu)
    ffc, fpos = (torch.randn(B, 128, 128, generator=g) / 11.0).to(gpu), torch.randn(B, 2, 128, generator=g).to(gpu)
    call = lambda: fused_encoder_tail_folded(q, pos, xr, ffc, fpos, bfc, w1, b1, w2, b2, "relu")
    assert torch.equal(on(main, call), on(check, call))


@pytest.mark.parametrize("K,N", [(128, 128), (136, 128), (128, 256), (256, 128), (70, 36), (32, 4), (128, 384), (200, 128),
                                 (132, 256), (1, 128), (20, 128), (32, 64)])
@pytest.mark.parametrize("T", [1, 63, 1000, 65536 + 3])
def test_linear_weight_grad(gpu, K, N, T):
    """dW = x^T g and db = column sums of g (the reference's projection backward, galerkin_attention.cu:41-46)
    against float64 products; ragged sizes, a strided x, and bit-identical reruns."""
    from spgt_amd.extension.bind.linear import linear_weight_grad
    gen = torch.Generator().manual_seed(K * 7 + N * 3 + T)
    xfull = torch.randn(T, K + 8, generator=gen)
    x, g = xfull[:, :K], torch.randn(T, N, generator=gen)
    xg = xfull.to(gpu)[:, :K]  # row stride K + 8
    dW, db = linear_weight_grad(xg, g.to(gpu))
    want_w, want_b = x.double().t() @ g.double(), g.double().sum(0)
    assert dW.shape == (K, N) and db.shape == (N,)
    scale = max(1.0, T ** 0.5)
    assert (dW.cpu().double() - want_w).abs().max() < 2e-5 * scale
    assert (db.cpu().double() - want_b).abs().max() < 2e-5 * scale
    dW2, db2 = linear_weight_grad(xg.contiguous(), g.to(gpu))
    assert torch.equal(dW, dW2) and torch.equal(db, db2)


def test_linear_weight_grad_batched_through_the_c_abi(gpu):
    """Three gradient planes against one input in one call (the packed Q | K | V projection's backward)."""
    import ctypes
    from spgt_amd import _lib
    lib = _lib.load()
    T, K, N = 5000, 128, 128
    gen = torch.Generator().manual_seed(5)
    x, g = torch.randn(T, K, generator=gen), torch.randn(3, T, N, generator=gen)
    xd, gd = x.to(gpu), g.to(gpu)
    out = torch.empty(3, K * N + N, device=gpu)
    nws = lib.spgt_linear_weight_grad_workspace_bytes(T, K, N, 3)
    ws = torch.empty(nws, dtype=torch.uint8, device=gpu)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    _lib.check(lib.spgt_linear_weight_grad(p(xd), K, 0, p(gd), N, T * N, p(out), p(ws), nws, T, K, N, 3,
                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    for j in range(3):
        assert (out[j, :K * N].view(K, N).cpu().double() - x.double().t() @ g[j].double()).abs().max() < 2e-3
        assert (out[j, K * N:].cpu().double() - g[j].double().sum(0)).abs().max() < 2e-3
    assert lib.spgt_linear_weight_grad_workspace_bytes(T, K, 126, 1) == 0


def test_dropout_add_and_its_backward(gpu):
    """residual + dropout(y) in one pass (the reference's F.dropout + residual add, network/sp_layer.py:76, 100-103,
    network/layer.py:173) with the library's own masks: kept values scaled by 1 / (1 - p), dropped ones leave the
    residual untouched, the kept fraction fits, another seed gives another mask; the autograd function's gradient of
    y carries the forward's mask and the residual's gradient is the incoming one."""
    from spgt_amd._lib import dropout_seed
    from spgt_amd.extension.bind.linear import dropout_add
    from spgt_amd.network.layer import always_dropout_add
    g = torch.Generator().manual_seed(3)
    p = 0.2
    y = torch.randn(5, 1000, 128, generator=g).to(gpu)
    r = torch.randn(5, 1000, 128, generator=g).to(gpu)
    seed = torch.tensor([5, 6], dtype=torch.int32, device=gpu)
    d = dropout_add(y, None, p, seed)
    keep = d != 0
    assert torch.equal(d[keep], (y * (1.0 / (1.0 - p)))[keep])
    assert keep.float().mean().item() == pytest.approx(1 - p, abs=3e-3)
    assert (keep[..., 1:] & keep[..., :-1]).float().mean().item() == pytest.approx((1 - p) ** 2, abs=4e-3)
    assert (keep[:, 1:] & keep[:, :-1]).float().mean().item() == pytest.approx((1 - p) ** 2, abs=4e-3)
    o = dropout_add(y, r, p, seed)
    assert torch.equal(o[~keep], r[~keep]) and torch.equal(o, d + r)
    other = dropout_add(y, None, p, torch.tensor([5, 7], dtype=torch.int32, device=gpu)) != 0
    assert (keep != other).float().mean().item() == pytest.approx(2 * p * (1 - p), abs=4e-3)
    assert (keep != (dropout_add(y, None, p, seed, site=6) != 0)).float().mean().item() == pytest.approx(
        2 * p * (1 - p), abs=4e-3)
    yg, rg = y.clone().requires_grad_(True), r.clone().requires_grad_(True)
    out = always_dropout_add(yg, rg, p)
    go = torch.randn(5, 1000, 128, generator=g).to(gpu)
    out.backward(go)
    kept = (out.detach() - r) != 0
    assert torch.equal(rg.grad, go)
    assert torch.equal(yg.grad[kept], (go * (1.0 / (1.0 - p)))[kept]) and (yg.grad[~kept] == 0).all()
    assert kept.float().mean().item() == pytest.approx(1 - p, abs=3e-3)
    alone = always_dropout_add(yg, None, p)
    assert alone.shape == y.shape and not torch.equal(alone, always_dropout_add(yg, None, p))
    assert torch.equal(always_dropout_add(y, r, 0.0), y + r)
