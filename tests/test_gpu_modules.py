"""The accelerated modules against golden vectors of the reference's plain-PyTorch modules
(converted state_dicts) and against the CPU oracle.  Attention-level outputs: max-rel <= 1e-4;
full-model output: relative L2 <= 1e-4."""
import pytest
import torch

from conftest import load_golden, max_rel, rel_l2
from oracle import spgt_oracle as O
from spgt_amd.network import model as M
from spgt_amd.network import sp_layer as L
from spgt_amd.network import sp_model as SM

pytestmark = pytest.mark.gpu
TOL = 1e-4


def load_into(module, params, gpu):
    missing, unexpected = module.load_state_dict(L.convert_gt_state_dict(params), strict=True)
    assert not missing and not unexpected
    return module.to(gpu).eval()


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_module_golden(gpu, dp):
    p, i, want, meta = load_golden(f"attention_dp{dp}")
    m = load_into(L.Sp_GalerkinAttention(128, int(meta["num_head"]), dp, float(meta["norm_eps"]), 0.0, 0.0, 1.0, 0.01,
                                         False), p, gpu)
    x, pos = i["x"].to(gpu), i["position"].to(gpu)
    with torch.no_grad():
        fused = m(x, x, x, pos)
        separate = m(x, x.clone(), x.clone(), pos)  # three GEMMs instead of the packed one
    assert max_rel(fused.cpu(), want) < TOL
    assert max_rel(separate.cpu(), want) < TOL
    graph_path = m(x, x, x, pos)  # autograd enabled: the reference's operator sequence
    assert max_rel(graph_path.detach().cpu(), want) < TOL


def test_encoder_layer_golden(gpu):
    p, i, want, meta = load_golden("encoder_layer")
    m = load_into(L.Sp_EncoderLayer(128, 4, 2, float(meta["norm_eps"]), 0.0, 0.0, 0.01, 0.01, False, 256, 0.0,
                                    str(meta["activation"])), p, gpu)
    with torch.no_grad():
        got = m(i["x"].to(gpu), i["position"].to(gpu))
    assert max_rel(got.cpu(), want) < TOL


def test_spectral_conv_golden(gpu):
    p, i, want, meta = load_golden("spectral_conv2d")
    m = load_into(L.Sp_SpectralConv2D(6, 4, int(meta["mode"]), 0.0, str(meta["activation"])), p, gpu)
    with torch.no_grad():
        got = m(i["x"].to(gpu))
    assert max_rel(got.cpu(), want) < TOL
    graph_path = m(i["x"].to(gpu))  # autograd enabled: gather, complex matmul, scatter
    assert max_rel(graph_path.detach().cpu(), want) < TOL
    m.use_truncated_dft = False  # inference through rfft2 / irfft2 and the full-spectrum contraction kernel
    with torch.no_grad():
        fft_path = m(i["x"].to(gpu))
    assert max_rel(fft_path.cpu(), want) < TOL


def test_scalers_golden(gpu):
    p, i, want, meta = load_golden("down_scaler")
    m = load_into(M.DownScaler2D(meta["resolution_size"].tolist(), 1, 128, 0.0, str(meta["activation"])), p, gpu)
    with torch.no_grad():
        got = m(i["x"].to(gpu))
    assert got.shape == want.shape and max_rel(got.cpu(), want) < TOL
    p, i, want, meta = load_golden("up_scaler")
    m = load_into(M.UpScaler2D(meta["resolution_size"].tolist(), 128, 128, 0.0, str(meta["activation"])), p, gpu)
    with torch.no_grad():
        got = m(i["x"].to(gpu))
    assert got.shape == want.shape and max_rel(got.cpu(), want) < TOL


def model_cfg(meta):
    cfg = {k: (v.item() if hasattr(v, "item") and getattr(v, "ndim", 1) == 0 else v) for k, v in meta.items()}
    cfg["resolution_size"] = meta["resolution_size"].tolist()
    cfg["target_normalizer"] = SM.UnitNormalizer()
    return cfg


def test_full_model_golden(gpu):
    p, i, want, meta = load_golden("galerkin_transformer_2d")
    m = load_into(SM.Sp_GalerkinTransformer2D(model_cfg(meta)), p, gpu)
    with torch.no_grad():
        got = m(i["x"].to(gpu), i["position"].to(gpu), i["grid"].to(gpu))
    assert got.shape == want.shape
    assert (got[:, 0] == 0).all() and (got[:, :, -1] == 0).all()
    assert rel_l2(got.cpu(), want) < TOL


def test_state_dict_layout_matches_reference(gpu):
    """Parameter names and shapes are the on-disk format; only weight orientation / Fourier layout differ."""
    p, _, _, meta = load_golden("galerkin_transformer_2d")
    m = SM.Sp_GalerkinTransformer2D(model_cfg(meta))
    sd = m.state_dict()
    assert set(sd.keys()) == set(p.keys())
    for k, v in L.convert_gt_state_dict(p).items():
        assert tuple(sd[k].shape) == tuple(v.shape), k
    fw = sd["decoder_regressor.layers.0.fourier_weight.0"]
    mode, width = int(meta["num_frequence_mode"]), int(meta["dim_spatial_hidden"])
    assert tuple(fw.shape) == (mode, mode, width, width, 2)


@pytest.mark.parametrize("r,ra", [(43, 22), (40, 12)])
def test_full_model_vs_oracle_mid_size(gpu, r, ra):
    """r = 43 -> r_attn = 22 with the resolution rule of the reference, and r = 40 -> 24 -> 12, where the up-scaler's
    convolution mixes channels before its interpolation; random init, against the oracle in fp64."""
    torch.manual_seed(3)
    rs = O.resolution_sizes(r, ra) if (r, ra) == (43, 22) else [[40, 40], [24, 24], [12, 12], [24, 24], [40, 40]]
    cfg = dict(
        drop_module=0.0, boundary_condition="dirichlet", target_normalizer=SM.UnitNormalizer(), resolution_size=rs,
        dim_node=1, dim_hidden=128, drop_downscaler=0.0, acti_downscaler="relu", num_encoder_layer=3, num_head=4,
        dim_position=2, attn_norm_eps=1e-6, drop_encoder_attn=0.0, drop_encoder_attn_fc=0.0, attn_xavier=0.5,
        attn_diagonal=0.01, attn_symmetric=False, dim_encoder_ffn=256, drop_encoder_ffn=0.0, acti_encoder_ffn="silu",
        drop_upscaler=0.0, acti_upscaler="silu", num_decoder_layer=2, dim_target=1, dim_spatial_hidden=64,
        num_frequence_mode=7, drop_decoder_layer=0.0, acti_decoder_layer="silu")
    m = SM.Sp_GalerkinTransformer2D(cfg)
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, r, r, 1, generator=g)
    lin = lambda n: torch.linspace(0, 1, n)
    mesh = lambda n: torch.stack(torch.meshgrid(lin(n), lin(n), indexing="ij"), dim=-1)[None].repeat(2, 1, 1, 1)
    pos, grid = mesh(ra), mesh(r)
    # oracle parameters: it computes x @ W^T with [Cin, Cout, m, m, 2] Fourier weights
    po = {}
    for k, v in sd.items():
        v = v.double()
        if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V"):
            v = v.t()
        po[k] = v
    want = O.galerkin_transformer_2d(po, cfg, x.double(), pos.double(), grid.double(), weight_layout="sp")
    m = m.to(gpu).eval()
    with torch.no_grad():
        got = m(x.to(gpu), pos.to(gpu), grid.to(gpu))
    assert rel_l2(got.cpu().double(), want) < TOL


def test_full_model_reference_yaml_defaults(gpu):
    """The reference's own default configuration (config/darcy_config.yaml with config_accessor.py:15-40 applied:
    R = 421, subsample_node 3 -> r = 141, subsample_attn 6 -> r_attn = 71, 6 encoder layers, spectral width 32,
    ceil(sqrt(141)) = 12 modes), drop rates 0, random init, against the oracle in fp64."""
    torch.manual_seed(5)
    r, ra = 141, 71
    cfg = dict(
        drop_module=0.0, boundary_condition="dirichlet", target_normalizer=SM.UnitNormalizer(),
        resolution_size=O.resolution_sizes(r, ra), dim_node=1, dim_hidden=128, drop_downscaler=0.0,
        acti_downscaler="relu", num_encoder_layer=6, num_head=4, dim_position=2, attn_norm_eps=1e-6,
        drop_encoder_attn=0.0, drop_encoder_attn_fc=0.0, attn_xavier=0.01, attn_diagonal=0.01, attn_symmetric=False,
        dim_encoder_ffn=256, drop_encoder_ffn=0.0, acti_encoder_ffn="relu", drop_upscaler=0.0, acti_upscaler="silu",
        num_decoder_layer=2, dim_target=1, dim_spatial_hidden=32, num_frequence_mode=12, drop_decoder_layer=0.0,
        acti_decoder_layer="silu")
    m = SM.Sp_GalerkinTransformer2D(cfg)
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    x = torch.randn(2, r, r, 1, generator=torch.Generator().manual_seed(6))
    lin = lambda n: torch.linspace(0, 1, n)
    mesh = lambda n: torch.stack(torch.meshgrid(lin(n), lin(n), indexing="ij"), dim=-1)[None].repeat(2, 1, 1, 1)
    pos, grid = mesh(ra), mesh(r)
    po = {k: (v.double().t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v.double())
          for k, v in sd.items()}
    want = O.galerkin_transformer_2d(po, cfg, x.double(), pos.double(), grid.double(), weight_layout="sp")
    m = m.to(gpu).eval()
    with torch.no_grad():
        got = m(x.to(gpu), pos.to(gpu), grid.to(gpu))
    assert rel_l2(got.cpu().double(), want) < TOL


@pytest.mark.parametrize("N,r,width,modes", [(1, 421, 32, 21), (1, 512, 32, 23), (2, 211, 64, 15), (2, 141, 32, 12)])
@pytest.mark.parametrize("truncated", [True, False])
def test_spectral_conv_reference_default_modes(gpu, N, r, width, modes, truncated):
    """Sp_SpectralConv2D at the mode counts config_accessor.py:39 derives (ceil(sqrt(r)): 21 at r = 421, 23 at 512,
    15 at 211, 12 at 141) and the yaml's width 32, both routes, against the oracle's rfft2 / irfft2 in fp64."""
    torch.manual_seed(7)
    layer = L.Sp_SpectralConv2D(width, width, modes, 0.0, "silu")
    with torch.no_grad():
        for w in layer.fourier_weight:
            w.copy_(torch.randn(w.shape) / width)
    sd = {k: v.clone().double() for k, v in layer.state_dict().items()}
    x = torch.randn(N, r, r, width, generator=torch.Generator().manual_seed(8))
    want = O.spectral_conv2d(sd, x.double(), modes, "silu", weight_layout="sp")
    layer = layer.to(gpu).eval()
    layer.use_truncated_dft = truncated
    with torch.no_grad():
        got = layer(x.to(gpu))
    assert max_rel(got.cpu().double(), want) < TOL


@pytest.mark.parametrize("N,r,cin,cout,modes", [(4, 256, 128, 32, 16), (2, 128, 128, 32, 12), (1, 512, 128, 32, 23),
                                                (2, 77, 128, 64, 9), (2, 50, 64, 32, 8)])
def test_spectral_conv_unequal_widths_take_the_fused_route(gpu, N, r, cin, cout, modes):
    """Sp_SpectralConv2D with in_dim != out_dim at the reference's own benchmark shape (evaluate/sp_fno2d.py:12-26:
    B = 4, 128 -> 32, modes ceil(sqrt(r))): the three-launch truncated-DFT route must serve it (no library GEMM or
    FFT behind it), and agree with the oracle's rfft2 / irfft2 in fp64."""
    from spgt_amd.network import truncated_dft
    torch.manual_seed(17)
    layer = L.Sp_SpectralConv2D(cin, cout, modes, 0.0, "silu")
    with torch.no_grad():
        for w in layer.fourier_weight:
            w.copy_(torch.randn(w.shape) / cin)
    sd = {k: v.clone().double() for k, v in layer.state_dict().items()}
    x = torch.randn(N, r, r, cin, generator=torch.Generator().manual_seed(18))
    want = O.spectral_conv2d(sd, x.double(), modes, "silu", weight_layout="sp")
    assert truncated_dft.fused_tail_supported(r, cin, cout, modes)
    layer = layer.to(gpu).eval()
    with torch.no_grad():
        got = layer(x.to(gpu))
    assert got.shape == (N, r, r, cout)
    assert max_rel(got.cpu().double(), want) < TOL


def test_deferred_upsampling_matches_module_order(gpu):
    """The decoder's input layer in front of the up-scaler's last interpolation (a Linear over the channels commutes
    with it) against the reference's order of the same modules (network/model.py:59-64, network/sp_model.py:60):
    grid values that are not a linear ramp, so that only the rank-2 grid update can place them."""
    p, i, _, meta = load_golden("galerkin_transformer_2d")
    m = load_into(SM.Sp_GalerkinTransformer2D(model_cfg(meta)), p, gpu)
    rs = meta["resolution_size"].tolist()
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, rs[2][0], rs[2][1], 128, generator=g).to(gpu)
    grid = torch.rand(2, rs[4][0], rs[4][1], 2, generator=g).to(gpu)
    up, dec = m.up_scaler, m.decoder_regressor
    with torch.no_grad():
        assert up.can_defer_last_resample(x)
        low = up(x, defer_last_resample=True)
        assert tuple(low.shape) == (2, rs[3][0], rs[3][1], 128) and dec.accepts_low_resolution(low, grid)
        want = dec(up(x), grid)
        got = dec(low, grid, resample_to=rs[4])
    assert got.shape == want.shape
    assert rel_l2(got.cpu(), want.cpu()) < 1e-5 and max_rel(got.cpu(), want.cpu()) < 1e-4


@pytest.mark.parametrize("act", ["silu", "relu"])
def test_up_scaler_mixing_before_resampling(gpu, act):
    """interpolate -> conv3x3 -> activations (network/model.py:59-62) computed as a GEMM on the low-resolution
    tokens plus a 9-tap gather, against the float64 oracle in the reference's order of operations; sizes with
    enough up-sampling for the fused path to choose this form (the golden vectors' sizes do not)."""
    torch.manual_seed(21)
    rs = [[20, 20], [14, 14], [8, 8], [14, 14], [20, 20]]
    m = M.UpScaler2D(rs, 128, 128, 0.0, act).eval()
    x = torch.randn(2, 8, 8, 128)
    want = O.up_scaler({k: v.double() for k, v in m.state_dict().items()}, x.double(), rs, act)
    with torch.no_grad():
        mg = m.to(gpu)
        xg = x.to(gpu)
        assert mg._mixes_before_resampling(xg)
        got = mg(xg)
        low = mg(xg, defer_last_resample=True)
    assert got.shape == want.shape and tuple(low.shape) == (2, 14, 14, 128)
    assert max_rel(got.cpu().double(), want) < 1e-5
    # the deferred form is the same tensor before the last interpolation
    from spgt_amd.extension.bind.datamove import bilinear_nhwc_affine
    assert torch.equal(bilinear_nhwc_affine(low, (20, 20)), got)


@pytest.mark.parametrize("dp,B,S", [(2, 3, 77), (0, 2, 200), (2, 1, 32), (2, 5, 1000), (0, 8, 19881), (2, 4, 5041),
                                     (2, 300, 33)])
def test_encoder_layer_folded_attention(gpu, dp, B, S):
    """The attention's Q.(K^T V / S) product folded into fc_layer's weight (associativity of network/sp_layer.py:64-75)
    against the unfolded fused layer; sequences whose length is not a multiple of the 32-token tile, and more
    workgroups than tiles as well as fewer."""
    torch.manual_seed(7)
    layer = L.Sp_EncoderLayer(128, 4, dp, 1e-6, 0.0, 0.0, 0.5, 0.01, False, 256, 0.0, "silu").to(gpu).eval()
    x = torch.randn(B, S, 128, device=gpu)
    pos = torch.rand(B, S, max(dp, 1), device=gpu)[:, :, :dp]
    with torch.no_grad():
        layer.fold_attention = False
        want = layer(x, pos)
        layer.fold_attention = True
        got = layer(x, pos)
        again = layer(x, pos)
        layer.fold_attention = None  # by size
        assert torch.equal(layer(x, pos), got if B * S >= layer.fold_attention_min_tokens else want)
    assert got.shape == want.shape and torch.equal(got, again)
    assert rel_l2(got.cpu(), want.cpu()) < 1e-5 and max_rel(got.cpu(), want.cpu()) < 1e-4


def test_dropout_seeds_of_one_forward_come_from_one_draw(gpu):
    """Inside a forward every dropout site gets its own word pair out of one generator call; outside, each
    call draws its own.  torch.manual_seed governs both."""
    from spgt_amd import _lib

    torch.manual_seed(5)
    with _lib.seed_scope():
        a, b = _lib.dropout_seed(gpu), _lib.dropout_seed(gpu)
        assert a.untyped_storage().data_ptr() == b.untyped_storage().data_ptr()
        assert a.data_ptr() + 8 == b.data_ptr() and a.numel() == b.numel() == 2
        pairs = [tuple(_lib.dropout_seed(gpu).tolist()) for _ in range(70)]  # runs past one pool
        assert len(set(pairs + [tuple(a.tolist()), tuple(b.tolist())])) == 72
    c = _lib.dropout_seed(gpu)
    assert c.numel() == 2 and c.untyped_storage().data_ptr() != a.untyped_storage().data_ptr()
    torch.manual_seed(5)
    with _lib.seed_scope():
        assert torch.equal(_lib.dropout_seed(gpu), a)


@pytest.mark.parametrize("fold", [False, True])
def test_encoder_layer_with_drop_rates_stays_fused(gpu, fold):
    """With the reference's drop rates (always on, F.dropout's default) the layer still runs as one launch after the
    attention core, with the two dropouts inside it.  A dropout only on fc_layer's output enters the layer's first
    residual sum linearly, so with the feed-forward net's second layer zeroed the mean over many draws is the layer
    without dropout; draws differ, torch.manual_seed repeats them, and a captured graph draws new masks on every
    replay."""
    torch.manual_seed(9)
    B, S = 2, 600
    layer = L.Sp_EncoderLayer(128, 4, 2, 1e-6, 0.0, 0.25, 0.5, 0.01, False, 256, 0.0, "relu").to(gpu).eval()
    layer.fold_attention = fold
    with torch.no_grad():
        layer.ffn_layer.layer2.weight.zero_()
        layer.ffn_layer.layer2.bias.zero_()
    x = torch.randn(B, S, 128, device=gpu)
    pos = torch.rand(B, S, 2, device=gpu)
    with torch.no_grad():
        layer.attention_layer.fc_droprate = 0.0
        want = layer(x, pos)
        layer.attention_layer.fc_droprate = 0.25
        n = 400
        acc = torch.zeros_like(want, dtype=torch.float64)
        for _ in range(n):
            acc += layer(x, pos)
        mean = (acc / n).float()
        # element-wise standard error of the mean: |term| sqrt(p / (1 - p) / n) = 0.029 |term|
        term = (want - x).abs()
        assert ((mean - want).abs() <= 0.029 * 6 * term + 1e-5).all()
        torch.manual_seed(3)
        a = layer(x, pos)
        b = layer(x, pos)
        torch.manual_seed(3)
        assert torch.equal(a, layer(x, pos)) and not torch.equal(a, b)
        layer.ffn_layer.droprate = 0.25
        c = layer(x, pos)
        assert torch.isfinite(c).all() and not torch.equal(c, a)
        # a captured forward: the seed words are drawn by a generator kernel inside the graph
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            layer(x, pos)
        torch.cuda.current_stream().wait_stream(stream)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = layer(x, pos)
        outs = []
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            outs.append(out.clone())
        assert not torch.equal(outs[0], outs[1]) and not torch.equal(outs[1], outs[2])


def test_model_with_the_reference_drop_rates(gpu):
    """The whole model with the yaml's drop rates (0.05 on the down-scaler's blocks, on fc_layer's output and on the
    feed-forward nets; the reference's dropouts are on in inference): the forward runs on the fused kernels with
    their own masks.  Two forwards differ, torch.manual_seed repeats one (up to the convolution library's own
    run-to-run rounding), and the mean over many forwards agrees with the mean over as many forwards of the same
    model on the route taken when gradients are enabled (other kernels, other launches, torch's F.dropout in the
    down-scaler's convolution blocks, separate dropout passes with seeds of their own elsewhere) as well as two such
    means agree with each other.  The masks' own properties are tested kernel by kernel."""
    p, i, _, meta = load_golden("galerkin_transformer_2d")
    cfgd = dict(model_cfg(meta), drop_downscaler=0.05, drop_encoder_attn_fc=0.05, drop_encoder_ffn=0.05)
    md = load_into(SM.Sp_GalerkinTransformer2D(cfgd), p, gpu)
    x, pos, grid = i["x"].to(gpu), i["position"].to(gpu), i["grid"].to(gpu)
    n = 300

    def mean_of(fn):
        acc = None
        for _ in range(n):
            y = fn().detach().double()
            acc = y if acc is None else acc + y
        return (acc / n).cpu()

    with torch.no_grad():
        torch.manual_seed(1)
        a = md(x, pos, grid)
        b = md(x, pos, grid)
        torch.manual_seed(1)
        again = md(x, pos, grid)
        assert rel_l2(again.cpu(), a.cpu()) < 1e-5 and rel_l2(b.cpu(), a.cpu()) > 1e-4
        fused = mean_of(lambda: md(x, pos, grid))
    with torch.enable_grad():
        ref1 = mean_of(lambda: md(x, pos, grid))
        ref2 = mean_of(lambda: md(x, pos, grid))
    noise = rel_l2(ref1, ref2)
    assert rel_l2(fused, ref1) < 2.0 * noise + 1e-3, (rel_l2(fused, ref1), noise)


def test_graphed_inference_replays_match_eager(gpu):
    """A HIP-graph capture of the whole forward: every replay, with eager work and synchronisation between
    replays and with fresh inputs, reproduces the eager forward.  The convolution library picks algorithms
    at this small size whose results vary from run to run in the last bits (two eager forwards differ by
    2e-6 of the output scale), so the comparison is at the path's 1e-4 and not bit for bit."""
    from spgt_amd.network.graphed import GraphedInference
    p, i, _, meta = load_golden("galerkin_transformer_2d")
    m = load_into(SM.Sp_GalerkinTransformer2D(model_cfg(meta)), p, gpu)
    x, pos, grid = i["x"].to(gpu), i["position"].to(gpu), i["grid"].to(gpu)
    g = GraphedInference(m, x, pos, grid)
    gen = torch.Generator().manual_seed(8)
    for rep in range(4):
        xr = x if rep == 0 else torch.randn(x.shape, generator=gen).to(gpu)
        with torch.no_grad():
            want = m(xr, pos, grid)
        torch.cuda.synchronize()
        got = g(xr, pos, grid).clone()
        torch.cuda.synchronize()
        assert rel_l2(got.cpu(), want.cpu()) < TOL, f"replay {rep} differs from the eager forward"
        _ = (torch.randn(257, 513, device=gpu) @ torch.randn(513, 129, device=gpu)).sum().item()  # eager work between replays
    with pytest.raises(ValueError):
        g(x[:1], pos, grid)


def test_parameters_changed_through_data_are_seen(gpu):
    """Writes through `.data` leave a parameter's version counter alone; the derived layouts the fused kernels read
    (transposed Linear weights, packed [W_Q | W_K | W_V], convolution taps, the split decoder input weight) must
    follow them all the same: forward, scale parameters in place, forward, compare with the oracle on the new values."""
    p, i, _, meta = load_golden("galerkin_transformer_2d")
    m = load_into(SM.Sp_GalerkinTransformer2D(model_cfg(meta)), p, gpu)
    x, pos, grid = i["x"].to(gpu), i["position"].to(gpu), i["grid"].to(gpu)
    cfg = dict(meta)
    cfg["resolution_size"] = meta["resolution_size"].tolist()

    def oracle_now():
        sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
        po = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
        return O.galerkin_transformer_2d(po, cfg, i["x"], i["position"], i["grid"], weight_layout="sp")

    with torch.no_grad():
        first = m(x, pos, grid)
    assert rel_l2(first.cpu(), oracle_now()) < TOL
    changed = 0
    for name, prm in m.named_parameters():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("weight_Q", "weight_V", "bias_K") or "fc_layer.weight" in name or "layer1.weight" in name or \
                "layer2.weight" in name or "up_scaler.conv.conv_layer.weight" in name or \
                "residual_layer.weight" in name:
            before = prm._version
            prm.data.mul_(1.5)
            prm.data.add_(0.01)
            assert prm._version == before  # nothing on the host records the write
            changed += 1
    assert changed >= 10
    with torch.no_grad():
        second = m(x, pos, grid)
    want = oracle_now()
    assert rel_l2(first.cpu(), want) > 1e-2  # the update matters
    assert rel_l2(second.cpu(), want) < TOL


def test_standalone_layers_follow_data_updates(gpu):
    """The same for layers used on their own, where no enclosing forward refreshes the derived layouts."""
    torch.manual_seed(5)
    layer = L.Sp_EncoderLayer(128, 4, 2, 1e-6, 0.0, 0.0, 0.5, 0.01, False, 256, 0.0, "silu").to(gpu).eval()
    x, pos = torch.randn(2, 300, 128, device=gpu), torch.rand(2, 300, 2, device=gpu)

    def oracle_now():
        sd = {k: v.detach().cpu().double() for k, v in layer.state_dict().items()}
        po = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
        return O.encoder_layer(po, x.cpu().double(), pos.cpu().double(), 4, 1e-6, "silu")

    for fold in (False, True):
        layer.fold_attention = fold
        with torch.no_grad():
            assert max_rel(layer(x, pos).cpu().double(), oracle_now()) < TOL
            layer.attention_layer.weight_K.data.mul_(-0.7)
            layer.attention_layer.fc_layer.weight.data.mul_(1.3)
            layer.ffn_layer.layer2.weight.data.add_(0.02)
            assert max_rel(layer(x, pos).cpu().double(), oracle_now()) < TOL
            # pieces called outside any forward refresh their own operands
            att = layer.attention_layer
            att.weight_Q.data.mul_(2.0)
            core = att.attend(x, x, x, pos)
            got = att.project(core, residual=x)
            sd = {k: v.detach().cpu().double() for k, v in att.state_dict().items()}
            po = {k: (v.t() if k in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
            want = x.cpu().double() + O.attention_module(po, x.cpu().double(), x.cpu().double(), x.cpu().double(),
                                                         pos.cpu().double(), 4, 1e-6)
            assert max_rel(got.cpu().double(), want) < TOL


def test_replaced_parameter_objects_are_seen(gpu):
    """A parameter that is replaced by another object (load_state_dict(assign=True), setattr) keeps the old tensor
    alive wherever it was captured; the derived layouts must be rebuilt from the module's current parameters.
    Forward, replace, forward, compare with the oracle on the new values; whole model and a layer on its own."""
    p, i, _, meta = load_golden("galerkin_transformer_2d")
    m = load_into(SM.Sp_GalerkinTransformer2D(model_cfg(meta)), p, gpu)
    x, pos, grid = i["x"].to(gpu), i["position"].to(gpu), i["grid"].to(gpu)
    cfg = dict(meta)
    cfg["resolution_size"] = meta["resolution_size"].tolist()

    def oracle_now():
        sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
        po = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
        return O.galerkin_transformer_2d(po, cfg, i["x"], i["position"], i["grid"], weight_layout="sp")

    with torch.no_grad():
        first = m(x, pos, grid)
    assert rel_l2(first.cpu(), oracle_now()) < TOL
    gen = torch.Generator().manual_seed(11)
    new_sd = {k: (v.detach().cpu() * 1.4 + 0.01 * torch.randn(v.shape, generator=gen)).to(gpu)
              for k, v in m.state_dict().items()}
    old_ptr = m.up_scaler.conv.conv_layer.weight.data_ptr()
    m.load_state_dict(new_sd, assign=True)
    assert m.up_scaler.conv.conv_layer.weight.data_ptr() != old_ptr
    with torch.no_grad():
        second = m(x, pos, grid)
    want = oracle_now()
    assert rel_l2(first.cpu(), want) > 1e-2
    assert rel_l2(second.cpu(), want) < TOL
    # setattr on single layers, outside any enclosing model forward
    torch.manual_seed(6)
    layer = L.Sp_EncoderLayer(128, 4, 2, 1e-6, 0.0, 0.0, 0.5, 0.01, False, 256, 0.0, "silu").to(gpu).eval()
    xs, ps = torch.randn(2, 300, 128, device=gpu), torch.rand(2, 300, 2, device=gpu)

    def layer_oracle():
        sd = {k: v.detach().cpu().double() for k, v in layer.state_dict().items()}
        po = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
        return O.encoder_layer(po, xs.cpu().double(), ps.cpu().double(), 4, 1e-6, "silu")

    with torch.no_grad():
        assert max_rel(layer(xs, ps).cpu().double(), layer_oracle()) < TOL
        att, ffn = layer.attention_layer, layer.ffn_layer
        att.weight_K = torch.nn.Parameter(att.weight_K.detach().clone() * -0.6)
        att.fc_layer.weight = torch.nn.Parameter(att.fc_layer.weight.detach().clone() * 1.2)
        ffn.layer1.weight = torch.nn.Parameter(ffn.layer1.weight.detach().t().contiguous().t() * 0.9)  # other strides
        assert max_rel(layer(xs, ps).cpu().double(), layer_oracle()) < TOL


def test_graphed_inference_follows_in_place_weight_updates(gpu):
    """A captured forward re-reads the parameters: after in-place updates (through the autograd-visible `copy_`
    and through `.data`), replays match eager forwards of the updated model."""
    from spgt_amd.network.graphed import GraphedInference
    p, i, _, meta = load_golden("galerkin_transformer_2d")
    m = load_into(SM.Sp_GalerkinTransformer2D(model_cfg(meta)), p, gpu)
    x, pos, grid = i["x"].to(gpu), i["position"].to(gpu), i["grid"].to(gpu)
    g = GraphedInference(m, x, pos, grid)
    with torch.no_grad():
        before = m(x, pos, grid).clone()
    torch.cuda.synchronize()
    assert rel_l2(g(x, pos, grid).cpu(), before.cpu()) < TOL
    for step in range(2):
        with torch.no_grad():
            for name, prm in m.named_parameters():
                if prm.dim() >= 2 and ("encoder_mixer" in name or "decoder_regressor" in name or "up_scaler" in name):
                    if step == 0:
                        prm.data.mul_(1.2)
                    else:
                        prm.copy_(prm * 0.9 + 0.003)
            want = m(x, pos, grid).clone()
        torch.cuda.synchronize()
        got = g(x, pos, grid).clone()
        torch.cuda.synchronize()
        assert rel_l2(want.cpu(), before.cpu()) > 1e-2
        assert rel_l2(got.cpu(), want.cpu()) < TOL, f"replay after update {step} used stale weights"


@pytest.mark.parametrize("dim_hidden,dp", [(256, 2), (384, 0), (512, 2), (640, 2), (768, 0)])
def test_attention_module_wider_models(gpu, dim_hidden, dp):
    """dim_hidden beyond 128 (the reference accepts any multiple of 128 with heads of 32, network/sp_layer.py:17):
    the inference path (library GEMM where the fused linear kernel has no variant, then the fused core), the
    packed self-attention form and the operator sequence under autograd, against the oracle in float64."""
    torch.manual_seed(9)
    H = dim_hidden // 32
    m = L.Sp_GalerkinAttention(dim_hidden, H, dp, 1e-6, 0.0, 0.0, 0.7, 0.01, False)
    with torch.no_grad():
        for prm in m.parameters():
            prm.add_(0.05 * torch.randn_like(prm))
    sd = {k: v.detach().double() for k, v in m.state_dict().items()}
    po = {k: (v.t() if k in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
    B, S = 2, 301
    x = torch.randn(B, S, dim_hidden)
    pos = torch.rand(B, S, max(dp, 1))[:, :, :dp]
    want = O.attention_module(po, x.double(), x.double(), x.double(), pos.double(), H, 1e-6)
    m = m.to(gpu).eval()
    xg, pg = x.to(gpu), pos.to(gpu)
    with torch.no_grad():
        packed = m(xg, xg, xg, pg)
        separate = m(xg, xg.clone(), xg.clone(), pg)
    operators = m(xg, xg, xg, pg)  # autograd on: projection operators + attention operator
    for got, name in ((packed, "packed"), (separate, "separate"), (operators.detach(), "operators")):
        assert max_rel(got.cpu().double(), want) < TOL, name


def test_unsupported_shapes_are_rejected_at_construction():
    with pytest.raises(ValueError):
        L.Sp_GalerkinAttention(128, 4, 1, 1e-6, 0.0, 0.0, 1.0, 0.0, False)
    L.Sp_GalerkinAttention(640, 20, 0, 1e-6, 0.0, 0.0, 1.0, 0.0, False)  # any multiple of 128, as the reference
