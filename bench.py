#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the fused Galerkin attention core (LayerNorm of K and V,
K^T V / S, Q (K^T V / S)) over one synthetic batch at the shape the metric is
quoted on: B=8, S=44521 (211 x 211 grid points), d_model=128, 4 heads, fp32,
inputs resident in HBM.  `value` is algorithmic bytes per second,
4*B*H*32*S*4 bytes (Q, K, V read once, out written once) per step.

One JSON line is printed.  Beside the contract keys it carries
  roofline      the kernel with the largest share of a call (the Q pass) against
                8 TB/s, timed with HIP events around the launch on its stream; the
                K/V pass and the whole call are reported inside it as well;
  cpu_baseline  the CPU oracle (restatement of the reference's plain PyTorch
                path) timed on this host's cores on the same shape;
  extra         secondary measurements: the feature-major attention operator, the
                config-2 split-K GEMM, every operator at its benchmark shape with
                rotated operands (kernel_rooflines), the workloads the reference
                itself published timings for (reference_published_shapes), and
                end-to-end Darcy inference (samples/s, with the CPU oracle of the
                same model timed beside it).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def cpu_baseline(B, S, H, seed, budget_s=20.0):
    """Oracle attention core on the host at the benchmark shape (fp32, all cores)."""
    import torch
    from oracle import spgt_oracle as O

    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(B, S, H * 32, generator=g) for _ in range(3))
    pos = torch.zeros(B, S, 0)
    one, zero = torch.ones(H, 32), torch.zeros(H, 32)
    run = lambda: O.attention_core_token_major(q, k, v, pos, one, zero, one, zero, 1e-6, H)
    with torch.no_grad():
        run()  # warm-up
        times = []
        t_start = time.perf_counter()
        while len(times) < 5 or (time.perf_counter() - t_start < budget_s and len(times) < 15):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
            if time.perf_counter() - t_start > 3 * budget_s:
                break
    times.sort()
    med = times[len(times) // 2]
    nbytes = 4 * B * H * 32 * S * 4
    return {
        "value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"oracle attention core (per-head layer_norm + stack + cat + 2 matmuls + head merge), fp32, "
                  f"full shape B={B} S={S} H={H}, median of {len(times)} runs, {med * 1e3:.1f} ms each",
        "ms_per_step": round(med * 1e3, 3),
    }


def max_rel_elementwise(got, want, floor=1e-3):
    """max |got - want| / |want| over the entries with |want| > floor * max|want|."""
    keep = want.abs() > floor * want.abs().max()
    return float(((got - want).abs()[keep] / want.abs()[keep]).max().item())


def darcy_inputs(B, r, r_attn, seed):
    """Synthetic Darcy batch: a = 12 where a Gaussian random field with covariance (-Laplace + 9 I)^-2
    is >= 0 and 3 elsewhere (the reference's dataset/darcy_generate recipe: alpha 2, tau 3, cosine
    basis, zero mean), plus the normalised coordinate grids at the fine and the attention resolution."""
    import numpy as np
    import torch
    from scipy.fft import idctn

    rng = np.random.default_rng(seed)
    k1, k2 = np.meshgrid(np.arange(r), np.arange(r), indexing="ij")
    coef = 3.0 * (np.pi ** 2 * (k1 ** 2 + k2 ** 2) + 9.0) ** (-1.0)  # tau^(alpha-1) (pi^2 |k|^2 + tau^2)^(-alpha/2)
    fields = []
    for _ in range(B):
        xi = rng.standard_normal((r, r))
        L = r * coef * xi
        L[0, 0] = 0.0
        g = idctn(L, type=2, norm="ortho")
        fields.append(np.where(g >= 0, 12.0, 3.0))
    a = torch.tensor(np.stack(fields), dtype=torch.float32)[..., None]
    lin = lambda n: torch.linspace(0, 1, n)
    mesh = lambda n: torch.stack(torch.meshgrid(lin(n), lin(n), indexing="ij"), dim=-1)[None].repeat(B, 1, 1, 1)
    return a, mesh(r_attn), mesh(r)


def darcy_config():
    """End-to-end configuration: reference architecture, sizes 211 -> 122 -> 71 -> 122 -> 211,
    4 encoder layers, FNO width 64, 12 modes, all drop rates 0."""
    return dict(
        drop_module=0.0, boundary_condition="dirichlet", resolution_size=((211, 211), (122, 122), (71, 71),
                                                                           (122, 122), (211, 211)),
        dim_node=1, dim_hidden=128, drop_downscaler=0.0, acti_downscaler="relu", num_encoder_layer=4, num_head=4,
        dim_position=2, attn_norm_eps=1e-6, drop_encoder_attn=0.0, drop_encoder_attn_fc=0.0, attn_xavier=0.01,
        attn_diagonal=0.01, attn_symmetric=False, dim_encoder_ffn=256, drop_encoder_ffn=0.0, acti_encoder_ffn="relu",
        drop_upscaler=0.0, acti_upscaler="silu", num_decoder_layer=2, dim_target=1, dim_spatial_hidden=64,
        num_frequence_mode=12, drop_decoder_layer=0.0, acti_decoder_layer="silu")


def darcy_bench(dev, with_cpu, steps=30, graph=True):
    """End-to-end Darcy inference, B=4, random init: samples/s on the GPU and, beside it, the CPU oracle."""
    import torch
    from spgt_amd.network import sp_model as SM

    B = 4
    cfg = darcy_config()
    torch.manual_seed(0)
    model = SM.Sp_GalerkinTransformer2D(dict(cfg, target_normalizer=SM.UnitNormalizer()))
    a, pos, grid = darcy_inputs(B, 211, 71, seed=0)
    sd = {k: v.clone() for k, v in model.state_dict().items()}
    model = model.to(dev).eval()
    ad, pd, gd = a.to(dev), pos.to(dev), grid.to(dev)
    from spgt_amd.network.graphed import GraphedInference
    with torch.no_grad():
        for _ in range(5):
            out = model(ad, pd, gd)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = model(ad, pd, gd)
        torch.cuda.synchronize()
        eager_ms = (time.perf_counter() - t0) / steps * 1e3
        if not graph:
            return {"ms_per_forward": round(eager_ms, 3), "samples_per_s": round(B / eager_ms * 1e3, 1), "batch": B,
                    "mode": "eager launches"}
        # the same forward replayed from a HIP graph: the coefficient field is copied into the captured buffer on
        # every call (a second tensor keeps that copy inside the timed region); the position and grid inputs are
        # constants of the model's resolution and live in the captured buffers
        graphed = GraphedInference(model, ad, pd, gd)
        a2 = ad.clone()
        pos_s, grid_s = graphed.static_inputs[1], graphed.static_inputs[2]
        for _ in range(3):
            gout = graphed(a2, pos_s, grid_s)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            gout = graphed(a2, pos_s, grid_s)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        graph_equal = bool(torch.equal(gout, out))
    graph_ms = ms
    res = {"ms_per_forward": round(eager_ms, 3), "samples_per_s": round(B / eager_ms * 1e3, 1), "batch": B,
           "mode": "eager launches (model(x, position, grid) as a user calls it); the HIP graph replay of the same "
                   "forward, input copy included, is reported separately",
           "eager_ms_per_forward": round(eager_ms, 3), "graph_ms_per_forward": round(graph_ms, 3),
           "graph_samples_per_s": round(B / graph_ms * 1e3, 1),
           "graph_output_equals_eager": graph_equal,
           "config": "r=211 -> 122 -> 71, 4 encoder layers (d_model 128, 4 heads, dp 2, FFN 256), "
                     "2 FNO blocks (width 64, 12 modes), random init, drop rates 0"}
    if with_cpu:
        from oracle import spgt_oracle as O
        po = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v) for k, v in sd.items()}
        with torch.no_grad():
            want = O.galerkin_transformer_2d(po, cfg, a, pos, grid, weight_layout="sp")  # warm-up + parity
            times = []
            for _ in range(3):
                t0 = time.perf_counter()
                O.galerkin_transformer_2d(po, cfg, a, pos, grid, weight_layout="sp")
                times.append(time.perf_counter() - t0)
        cpu_ms = sorted(times)[1] * 1e3
        res["cpu_oracle_ms_per_forward"] = round(cpu_ms, 1)
        res["cpu_oracle_samples_per_s"] = round(B / cpu_ms * 1e3, 2)
        res["cpu_cores"] = torch.get_num_threads()
        res["rel_l2_vs_cpu_oracle"] = float(((out.cpu() - want).norm() / want.norm()).item())
        res["max_rel_elementwise_vs_cpu_oracle"] = max_rel_elementwise(out.cpu(), want)
    return res


def _gpu_ms(fn, steps, warm=3):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def _cpu_ms(fn, runs=3):
    fn()
    times = []
    for _ in range(runs):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2] * 1e3


def encoder_stack_bench(dev, with_cpu):
    """Config 3: 6 encoder layers (d_model 128, 4 heads, K/V LayerNorm, FFN 128-256-128 SiLU, dp 0),
    input [8, 19881, 128] ~ N(0,1), Xavier-uniform projections (gain 1), biases 0."""
    import torch
    from spgt_amd.network import sp_layer as L

    B, S, nl = 8, 19881, 6
    torch.manual_seed(0)
    layers = [L.Sp_EncoderLayer(128, 4, 0, 1e-6, 0.0, 0.0, 1.0, 0.0, False, 256, 0.0, "silu") for _ in range(nl)]
    for layer in layers:
        for name, prm in layer.named_parameters():
            if name.endswith("bias") and prm.dim() == 1:
                torch.nn.init.zeros_(prm)
    sds = [{k: v.clone() for k, v in layer.state_dict().items()} for layer in layers]
    x = torch.randn(B, S, 128, generator=torch.Generator().manual_seed(0))
    pos = torch.zeros(B, S, 0)
    mods = [layer.to(dev).eval() for layer in layers]
    xd, pd = x.to(dev), pos.to(dev)

    def fwd():
        y = xd
        for m in mods:
            y = m(y, pd)
        return y

    with torch.no_grad():
        ms = _gpu_ms(fwd, 10)
        out = fwd()
    res = {"ms_per_forward": round(ms, 3), "samples_per_s": round(B / ms * 1e3, 1), "batch": B}
    if with_cpu:
        from oracle import spgt_oracle as O
        pos_c = pos

        def cpu_fwd():
            y = x
            for sd in sds:
                po = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v)
                      for k, v in sd.items()}
                y = O.encoder_layer(po, y, pos_c, 4, 1e-6, "silu")
            return y

        with torch.no_grad():
            cpu_ms = _cpu_ms(cpu_fwd)
            want = cpu_fwd()
        res.update(cpu_oracle_ms_per_forward=round(cpu_ms, 1), cpu_cores=torch.get_num_threads(),
                   rel_l2_vs_cpu_oracle=float(((out.cpu() - want).norm() / want.norm()).item()),
                   max_rel_elementwise_vs_cpu_oracle=max_rel_elementwise(out.cpu(), want))
    return res


def fno_stack_bench(dev, with_cpu):
    """Config 4: 4 spectral-conv blocks, width 64, 12 modes, input [8, 141, 141, 64] ~ N(0,1), Fourier weights
    U[0, 1/(64*64)); the reference module's activation choices are silu|relu, SiLU is used."""
    import torch
    from spgt_amd.network import sp_layer as L

    B, r, C, m, nl = 8, 141, 64, 12, 4
    torch.manual_seed(0)
    layers = [L.Sp_SpectralConv2D(C, C, m, 0.0, "silu") for _ in range(nl)]
    g = torch.Generator().manual_seed(0)
    for layer in layers:
        with torch.no_grad():
            for w in layer.fourier_weight:
                w.copy_(torch.rand(w.shape, generator=g) / (C * C))
    sds = [{k: v.clone() for k, v in layer.state_dict().items()} for layer in layers]
    x = torch.randn(B, r, r, C, generator=g)
    mods = [layer.to(dev).eval() for layer in layers]
    xd = x.to(dev)

    def fwd():
        y = xd
        for mod in mods:
            y = mod(y)
        return y

    with torch.no_grad():
        ms = _gpu_ms(fwd, 10)
        out = fwd()
    res = {"ms_per_forward": round(ms, 3), "samples_per_s": round(B / ms * 1e3, 1), "batch": B}
    if with_cpu:
        from oracle import spgt_oracle as O

        def cpu_fwd():
            y = x
            for sd in sds:
                y = O.spectral_conv2d(sd, y, m, "silu", weight_layout="sp")
            return y

        with torch.no_grad():
            cpu_ms = _cpu_ms(cpu_fwd)
            want = cpu_fwd()
        res.update(cpu_oracle_ms_per_forward=round(cpu_ms, 1), cpu_cores=torch.get_num_threads(),
                   rel_l2_vs_cpu_oracle=float(((out.cpu() - want).norm() / want.norm()).item()),
                   max_rel_elementwise_vs_cpu_oracle=max_rel_elementwise(out.cpu(), want))
    return res


ROTATE_BYTES = 512 * 1024 * 1024  # traffic that must pass between two uses of one operand set
MAX_SETS = 24


class Rotation:
    """Times one operator over several independent operand sets visited in turn, so that no call finds its
    inputs, or the lines it writes, in the 256 MB last-level cache: between two uses of a set at least
    ROTATE_BYTES of other sets' traffic pass (as far as MAX_SETS sets allow; `bytes_between_reuse` says how
    much it was).  Outputs of the last round are kept alive, so the allocator hands every call other memory.
    The same operator on one set, outputs reused, is timed beside it (`us_one_set`)."""

    def __init__(self, dev, use_graph):
        self.dev, self.use_graph = dev, use_graph

    def _time(self, seq, n, replays=5):
        import torch
        for i in range(min(n, 6)):
            seq(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        mode = "eager"
        if self.use_graph:
            # n calls captured into a HIP graph and replayed: short kernels are timed on the GPU's clock and not
            # on the host's launch rate.  torch.cuda.graph ends the capture also when the body raises.
            graph = torch.cuda.CUDAGraph()
            try:
                with torch.cuda.graph(graph):
                    for i in range(n):
                        seq(i)
                mode = "graph"
            except RuntimeError:
                torch.cuda.synchronize()
                graph = None
        if mode == "graph":
            graph.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(replays):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) / (n * replays) * 1e-3
            del graph
            return t, mode
        e0.record()
        for i in range(n):
            seq(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e-3, mode

    def run(self, make, traffic_bytes):
        """make() builds one fresh operand set and returns a callable over it.  -> dict of timings."""
        import collections
        import math
        import torch
        nsets = max(2, min(MAX_SETS, math.ceil(ROTATE_BYTES / max(1, traffic_bytes)) + 1))
        fns = [make() for _ in range(nsets)]
        keep = collections.deque(maxlen=nsets)
        n = nsets * max(1, math.ceil(20 / nsets))
        t_rot, mode = self._time(lambda i: keep.append(fns[i % nsets]()), n)
        keep.clear()
        t_one, mode_one = self._time(lambda i: fns[0](), 20)
        del fns
        torch.cuda.empty_cache()
        return {"t": t_rot, "t_one": t_one, "sets": nsets, "between": (nsets - 1) * traffic_bytes,
                "mode": mode if mode == mode_one else f"{mode}/{mode_one}"}


def kernel_rooflines(dev, use_graph=True):
    """Every operator of the path at its benchmark shape: algorithmic bytes (or flops), time from HIP events on the
    launch stream, and the fraction of the bounding peak (HBM 8 TB/s; fp32 MFMA 157.3 TFLOP/s).  Operands rotate
    (see Rotation): `us` and the fractions are figures with inputs and outputs coming from and going to HBM;
    `us_one_set` is the same call repeated on one operand set.  A row whose operand sets could not be rotated far
    enough (tiny windows of large tensors) carries frac_hbm = null and says so.  use_graph=False launches eagerly
    (for runs under a profiler, which then sees plain dispatches)."""
    import torch
    from spgt_amd.extension.bind import datamove as dm
    from spgt_amd.extension.bind import galerkin_attention as ga
    from spgt_amd.extension.bind import linear as ln

    rot = Rotation(dev, use_graph)
    rows = {}
    # eager runs (under a profiler): one fill kernel before every row, so that a trace can be cut into rows
    marker = None if use_graph else torch.zeros(64, dtype=torch.int16, device=dev)  # no other int16 fill in the run

    def mark():
        if marker is not None:
            marker.fill_(len(rows))

    def common(r):
        return {"us": round(r["t"] * 1e6, 2), "us_one_set": round(r["t_one"] * 1e6, 2), "operand_sets": r["sets"],
                "bytes_between_reuse": int(r["between"]), "timing": r["mode"]}

    def hbm(name, nbytes, make, traffic=None):
        mark()
        r = rot.run(make, traffic if traffic is not None else nbytes)
        row = common(r)
        ok = r["between"] >= ROTATE_BYTES
        row.update({"bytes": int(nbytes), "GB/s": round(nbytes / r["t"] / 1e9, 1),
                    "frac_hbm": round(nbytes / r["t"] / 1e9 / HBM_PEAK_GBPS, 4) if ok else None})
        if not ok:
            row["note"] = "operand windows too small to rotate out of the last-level cache: a latency figure"
        rows[name] = row

    def mfma(name, flops, nbytes, make):
        mark()
        r = rot.run(make, nbytes)
        row = common(r)
        row.update({"flops": int(flops), "TFLOP/s": round(flops / r["t"] / 1e12, 2),
                    "frac_mfma_f32": round(flops / r["t"] / 1e12 / 157.3, 4)})
        rows[name] = row

    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *shape: torch.randn(*shape, device=dev, generator=g)
    ru = lambda *shape: torch.rand(*shape, device=dev, generator=g)
    B, S, H = 8, 44521, 4
    one, zero = torch.ones(H, 32, device=dev), torch.zeros(H, 32, device=dev)
    W, bias = rn(128, 128) / 11.3, rn(128)

    def fused(dp):
        def make():
            q, k, v = rn(B, S, 128), rn(B, S, 128), rn(B, S, 128)
            pos = ru(B, S, 2) if dp else None
            return lambda: ga.galerkin_attention_fused(q, k, v, pos, one, zero, one, zero, 1e-6, H, dp)
        return make

    hbm("attention_fused_dp0", 4 * B * S * 128 * 4, fused(0))
    hbm("attention_fused_dp2", (3 * 128 + 136 + 2 * 2) * B * S * 4, fused(2))

    # backward of the fused core: grad_out, q, k, v read, dq, dk, dv written (each counted once; the kernel
    # reads grad_out twice), LayerNorm backward of K and V included
    def fused_bwd(dp):
        def make():
            q, k, v = rn(B, S, 128), rn(B, S, 128), rn(B, S, 128)
            pos = ru(B, S, 2) if dp else None
            G = rn(B, S, H * (32 + dp))
            ktv = rn(B, H, 32 + dp, 32 + dp)
            return lambda: ga.gexts.galerkin_attention_fused_backward(G, q, k, v, pos, one, zero, one, zero, 1e-6, ktv,
                                                                      H, dp)
        return make
    hbm("attention_fused_backward_dp0", 7 * B * S * 128 * 4, fused_bwd(0))
    hbm("attention_fused_backward_dp2", (6 * 128 + 136 + 2) * B * S * 4, fused_bwd(2))

    def projection(layernorm, dp):
        def make():
            x, pos = rn(B, S, 128), ru(B, S, 2)[..., :dp]
            if layernorm:
                return lambda: ga.multihead_projection_layernorm_with_position_rrc_cuda(x, W, bias, one, zero, pos, 1e-6,
                                                                                        H, 32, dp)
            return lambda: ga.multihead_projection_with_position_rrc_cuda(x, W, bias, pos, H, 32, dp)
        return make

    proj_bytes = lambda dp: B * S * (128 + H * (32 + dp)) * 4
    mfma("projection_rrc_dp0", 2 * B * S * 128 * 128, proj_bytes(0), projection(False, 0))
    mfma("projection_layernorm_rrc_dp2", 2 * B * S * 128 * 128, proj_bytes(2), projection(True, 2))
    for d in (32, 34):
        def make(d=d):
            Qf, Kf, Vf = rn(B, H, d, S), rn(B, H, d, S), rn(B, H, d, S)
            return lambda: ga.multihead_galerkin_attention_cccr_cuda(Qf, Kf, Vf)
        hbm(f"attention_cccr_d{d}", 4 * B * H * d * S * 4, make)

        # backward of the operator: reads grad_out, Q, K, V, writes dQ, dK, dV (7 tensors of B*H*d*S floats)
        def make_bwd(d=d):
            Qf, Kf, Vf, G = rn(B, H, d, S), rn(B, H, d, S), rn(B, H, d, S), rn(B, H, S, d)
            return lambda: ga.gexts.multihead_galerkin_attention_cccr_backward(G, Qf, Kf, Vf, B, H, d, S)
        hbm(f"attention_cccr_backward_d{d}", 7 * B * H * d * S * 4, make_bwd)

    # LayerNorm backward of the projection+LayerNorm operator (per-head statistics recomputed from the
    # pre-LayerNorm projection): reads pre and grad, writes grad_pre; dgamma, dbeta by fixed-order sums
    def make_lnb():
        import ctypes
        from spgt_amd import _lib
        lib = _lib.load()
        T = B * S
        pre, gr, out = rn(T, 128), rn(T, 128), torch.empty(T, 128, device=dev)
        gw, gb = torch.empty(H, 32, device=dev), torch.empty(H, 32, device=dev)
        nws = lib.spgt_layernorm_heads_backward_workspace_bytes(T, H)
        ws = torch.empty(max(16, nws), dtype=torch.uint8, device=dev)
        p = lambda t: ctypes.c_void_p(t.data_ptr())

        def call():
            rc = lib.spgt_layernorm_heads_backward(p(pre), p(gr), p(one), 1e-6, p(out), p(gw), p(gb), p(ws), ws.numel(),
                                                   T, H, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            if rc != 0:
                raise RuntimeError("layernorm_heads_backward failed")
            return out
        return call
    hbm("layernorm_heads_backward", 3 * B * S * 128 * 4, make_lnb)

    def make_c2():
        A, Bm = rn(32, 32, S), rn(32, S, 32)
        return lambda: ga.batched_skinny_gemm(A, Bm, 1.0)
    hbm("batched_skinny_gemm_config2", 2 * 32 * 32 * S * 4 + 32 * 32 * 32 * 4, make_c2)

    # FNO path at config 4: N=8, C=64, r=141, m=12
    N, C, r, m = 8, 64, 141, 12
    wa = r // 2 + 1
    act_bytes = N * r * r * C * 4

    def make_t1():
        x = rn(N, r, r, C)
        return lambda: dm.batched_transpose(x, [N], [r, r], [C])

    def make_t2():
        xt = rn(N, C, r, r)
        return lambda: dm.batched_transpose(xt, [N], [C], [r, r])
    hbm("batched_transpose_nhwc_to_nchw", 2 * act_bytes, make_t1)
    hbm("batched_transpose_nchw_to_nhwc", 2 * act_bytes, make_t2)
    w0, w1 = ru(m, m, C, C, 2) / (C * C), ru(m, m, C, C, 2) / (C * C)

    def make_gather():
        xf = torch.view_as_complex(rn(N, C, r, wa, 2))
        return lambda: dm.transpose_gather_dual(xf, [N, C], r, wa, m, m, 0, 0, r - m, 0)
    hbm("transpose_gather_dual", 2 * 2 * m * m * N * C * 8, make_gather)

    def make_scatter():
        g0, g1 = (torch.view_as_complex(rn(m, m, N, C, 2)) for _ in range(2))
        return lambda: dm.transpose_scatter_dual(g0, g1, [N, C], r, wa, m, m, 0, 0, r - m, 0)
    hbm("transpose_scatter_dual", 2 * m * m * N * C * 8 + N * C * r * wa * 8, make_scatter)

    def make_contract():
        xf = torch.view_as_complex(rn(N, C, r, wa, 2))
        return lambda: dm.spectral_mode_contract(xf, w0, w1, m, m, 0, 0, r - m, 0)
    hbm("spectral_mode_contract", 2 * m * m * 8 * (N * C + C * C + N * C) + N * C * r * wa * 8, make_contract)

    # resampling at the Darcy model's sizes (B=4, 128 channels, 211 / 122 / 71)
    cb = rn(128)
    bil = lambda a, b: 4 * 4 * 128 * (a * a + b * b)

    def resample(shape, fn):
        def make():
            t = rn(*shape)
            return lambda: fn(t)
        return make

    hbm("bilinear_211_to_122", bil(211, 122), resample((4, 128, 211, 211), lambda t: dm.bilinear_align_corners(t, (122, 122))))
    hbm("bilinear_71_to_122", bil(71, 122), resample((4, 128, 71, 71), lambda t: dm.bilinear_align_corners(t, (122, 122))))
    hbm("bilinear_122_to_211_nchw_to_nhwc", bil(122, 211),
        resample((4, 128, 122, 122), lambda t: dm.bilinear_resample(t, (211, 211), dst_nhwc=True)))
    hbm("bilinear_122_to_71_nchw_to_nhwc", bil(122, 71),
        resample((4, 128, 122, 122), lambda t: dm.bilinear_resample(t, (71, 71), dst_nhwc=True)))
    hbm("bilinear_71_to_122_nhwc_to_nchw", bil(71, 122),
        resample((4, 71, 71, 128), lambda t: dm.bilinear_resample(t, (122, 122), src_nhwc=True)))

    def make_affine():
        low64, grid2, wg = rn(4, 122, 122, 64), rn(4, 211, 211, 2), rn(2, 64)
        return lambda: dm.bilinear_nhwc_affine(low64, (211, 211), grid2, wg)
    hbm("bilinear_122_to_211_nhwc_plus_grid_columns", 4 * 4 * (64 * (211 * 211 + 122 * 122) + 2 * 211 * 211), make_affine)
    # the resampling's backward (a gather per source position), planes and channels-last
    hbm("bilinear_adjoint_122_to_211_planes", bil(211, 122),
        resample((4, 128, 122, 122), lambda t: dm.bilinear_adjoint(t, (211, 211))))
    hbm("bilinear_adjoint_211_to_122_nhwc", bil(122, 211),
        resample((4, 211, 211, 128), lambda t: dm.bilinear_adjoint(t, (122, 122), nhwc=True)))
    hbm("bias_silu2_nchw_to_nhwc_122", 2 * 4 * 128 * 122 * 122 * 4,
        resample((4, 128, 122, 122), lambda t: dm.bilinear_resample(t, (122, 122), dst_nhwc=True, pre_bias=cb,
                                                                     pre_activation="silu", pre_count=2)))
    hbm("bilinear_211_to_122_bias_silu_silu", bil(211, 122),
        resample((4, 128, 211, 211), lambda t: dm.bilinear_resample(t, (122, 122), pre_activation="silu",
                                                                     post_activation="silu", pre_bias=cb)))
    hbm("bias_activation_nchw_silu2", 2 * 4 * 128 * 122 * 122 * 4,
        resample((4, 128, 122, 122), lambda t: dm.bias_activation_nchw_(t, cb, "silu", 2)))

    # fused linear layers at the encoder's and the decoder's token counts of the Darcy model
    w3, b3 = rn(128, 384) / 11.3, rn(384)
    w4, b4 = rn(128, 256) / 11.3, rn(256)
    w5 = rn(256, 128) / 16.0
    wfc = rn(136, 128) / 11.7
    for T, tag in ((B * S, "356k"), (4 * 71 * 71, "20k")):
        def lin(k, fn, extra_res=False):
            def make():
                x = rn(T, k)
                res = rn(T, 128) if extra_res else None
                return lambda: fn(x, res)
            return make
        mfma(f"linear_128_to_128_T{tag}", 2 * T * 128 * 128, T * 256 * 4, lin(128, lambda x, _: ln.fused_linear(x, W, bias)))
        mfma(f"linear_qkv_128_to_384_planes_T{tag}", 2 * T * 128 * 384, T * 512 * 4,
             lin(128, lambda x, _: ln.fused_linear(x, w3, b3, planes=3)))
        mfma(f"linear_128_to_256_silu_T{tag}", 2 * T * 128 * 256, T * 384 * 4,
             lin(128, lambda x, _: ln.fused_linear(x, w4, b4, "silu")))
        mfma(f"linear_256_to_128_residual_T{tag}", 2 * T * 256 * 128, T * 512 * 4,
             lin(256, lambda x, res: ln.fused_linear(x, w5, bias, "none", res), True))
        # an encoder layer after the attention core in one launch (output projection 136 -> 128, residuals, FFN 256)
        mfma(f"encoder_tail_136_128_256_T{tag}", 2 * T * (136 * 128 + 2 * 128 * 256), T * (136 + 256) * 4,
             lin(136, lambda x, res: ln.fused_encoder_tail(x, res, wfc, bias, w4, b4, w5, bias, "silu"), True))
    # weight + bias gradient of a Linear from token-major x and dL/dy (one pass over both, fixed summation order)
    for T, tag in ((B * S, "356k"), (4 * 128 * 128, "65k")):
        def make_wgrad():
            x, gy = rn(T, 128), rn(T, 128)
            return lambda: ln.linear_weight_grad(x, gy)
        mfma(f"linear_weight_grad_128x128_T{tag}", 2 * T * 128 * 128, T * 256 * 4, make_wgrad)
    Tf = 4 * 211 * 211
    w6, b6 = rn(64, 64) / 8.0, rn(64)
    w7, b7, w8, b8 = rn(64, 256) / 8.0, rn(256), rn(1, 256) / 16.0, rn(1)

    def make_l64():
        x, y = rn(Tf, 64), rn(Tf, 64)
        return lambda: ln.fused_linear(x, w6, b6, "silu", y)

    def make_ffn():
        x = rn(Tf, 64)
        return lambda: ln.fused_ffn_scalar(x, w7, b7, w8, b8, "silu")
    mfma("linear_64_to_64_residual_silu_T178k", 2 * Tf * 64 * 64, Tf * 192 * 4, make_l64)
    mfma("ffn_scalar_64_256_1_T178k", 2 * Tf * 64 * 256 + 2 * Tf * 256, Tf * 65 * 4, make_ffn)
    # truncated DFT along w at the decoder's grid: rows = 4*211, r = 211, C = 64, 12 modes
    from spgt_amd.network.truncated_dft import dft_tables
    fw, _, _, fwi = dft_tables(211, 12, dev)
    dft_bytes = (Tf * 64 + 4 * 211 * 64 * 24) * 4

    def make_dftf():
        x = rn(4 * 211, 211, 64)
        return lambda: dm.truncated_dft_rows_forward(x, fw)

    def make_dfti():
        u = rn(4 * 211, 64, 24)
        return lambda: dm.truncated_dft_rows_inverse(u, fwi)
    hbm("truncated_dft_rows_forward", dft_bytes, make_dftf)
    hbm("truncated_dft_rows_inverse", dft_bytes, make_dfti)
    return rows


def reference_published_shapes(dev, quick=False):
    """The workloads the reference itself timed (evaluate/sp_all.py:8-19 -> sp_galerkin.py, sp_fno2d.py,
    sp_darcy_breakdown.py, sp_darcy_ablation.py), at the shapes of its published tables, each beside the
    published V100-SXM2 / RTX 4090 figure (storage/evaluation/time.tgz; context, not a like-for-like
    comparison: other hardware).  Inputs are torch.rand as there; operand sets rotate so that ~512 MB pass
    between two uses of a set; HIP events around every call, median and p10 / p90 in microseconds.
    Where the reference timed a forward with requires_grad inputs (its modules then record an autograd
    graph), that form is reported as `..._grad_enabled` next to the inference form (torch.no_grad)."""
    import math
    import torch
    from spgt_amd.extension.bind import galerkin_attention as ga
    from spgt_amd.network import model as M
    from spgt_amd.network import sp_layer as L
    from spgt_amd.network import sp_model as SM

    ru = lambda *shape, **kw: torch.rand(*shape, device=dev, **kw)
    out = {}

    def stats(times_ms):
        vs = sorted(times_ms)
        pick = lambda f: vs[min(len(vs) - 1, int(f * len(vs)))]
        return {"median_us": round(pick(0.5) * 1e3, 1), "p10_us": round(pick(0.1) * 1e3, 1),
                "p90_us": round(pick(0.9) * 1e3, 1), "calls": len(vs)}

    def timed(fns, n=None, warm=3):
        """fns: callables over independent operand sets, visited in turn."""
        n = n or (8 if quick else max(12, 3 * len(fns)))
        keep = []
        for i in range(warm):
            keep.append(fns[i % len(fns)]())
        keep.clear()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for i, (e0, e1) in enumerate(evs):
            e0.record()
            r = fns[i % len(fns)]()
            e1.record()
            keep.append(r)
            if len(keep) > len(fns):
                keep.pop(0)
        torch.cuda.synchronize()
        keep.clear()
        return stats([e0.elapsed_time(e1) for e0, e1 in evs])

    def nsets(traffic_bytes):
        return max(2, min(8, math.ceil(ROTATE_BYTES / traffic_bytes) + 1))

    def row(name, st, published, **more):
        st = dict(st)
        st["published_us"] = published
        st.update(more)
        out[name] = st
        torch.cuda.empty_cache()

    # ---- batched skinny GEMM [16, 32, S] x [16, S, 32] (sp_galerkin.py:20-72) ----
    for S_, pub in ((65536, {"V100 exts": 511.6, "V100 torch.matmul": 5156.4, "RTX4090 exts": 378.9}),
                    (262144, {"V100 exts": 2043.0, "V100 torch.matmul": 21035.4, "RTX4090 exts": 1570.5})):
        nb = 2 * 16 * 32 * S_ * 4
        sets = [(ru(16, 32, S_), ru(16, S_, 32)) for _ in range(nsets(nb))]
        st = timed([lambda a=a, b=b: ga.batched_skinny_gemm(a, b) for a, b in sets])
        lib = timed([lambda a=a, b=b: torch.matmul(a, b) for a, b in sets])
        row(f"skinny_gemm_16x32x{S_}", st, pub, GBps=round(nb / st["median_us"] / 1e3, 1),
            frac_hbm=round(nb / st["median_us"] / 1e3 / HBM_PEAK_GBPS, 4), torch_matmul_here_us=lib["median_us"])
        del sets

    # ---- projection + position, projection + LayerNorm + position, B=16, S=65536, dp=2 (sp_galerkin.py:130-229) ----
    Bp, Sp, Hh = 16, 65536, 4
    W, b = ru(128, 128, requires_grad=True), ru(128, requires_grad=True)
    lw, lb = ru(Hh, 32, requires_grad=True), ru(Hh, 32, requires_grad=True)
    psets = [(ru(Bp, Sp, 128, requires_grad=True), ru(Bp, Sp, 2)) for _ in range(2)]
    flops = 2 * Bp * Sp * 128 * 128
    proj = lambda x, pos: ga.multihead_projection_with_position_rrc_cuda(x, W, b, pos, Hh, 32, 2)
    projln = lambda x, pos: ga.multihead_projection_layernorm_with_position_rrc_cuda(x, W, b, lw, lb, pos, 1e-5, Hh, 32, 2)
    for name, fn, pub_f, pub_b, wrt in (
            ("projection_position", proj, {"V100 exts": 2878.4, "V100 torch": 12242.5, "RTX4090 exts": 1668.9},
             {"V100 exts": 7684.7, "RTX4090 exts": 4178.7}, lambda x: [x, W, b]),
            ("projection_layernorm_position", projln,
             {"V100 exts": 5413.1, "V100 torch": 29096.0, "RTX4090 exts": 2701.4},
             {"V100 exts": 15457.2, "RTX4090 exts": 7306.4}, lambda x: [x, W, b, lw, lb])):
        st = timed([lambda x=x, pos=pos: fn(x, pos) for x, pos in psets])
        row(f"{name}_forward_B16_S65536_dp2", st, pub_f, TFLOPs=round(flops / st["median_us"] / 1e6, 1))
        ys = [fn(x, pos) for x, pos in psets]
        gs = [torch.rand_like(y) for y in ys]
        st = timed([lambda x=x, y=y, g=g: torch.autograd.grad(outputs=y, inputs=wrt(x), grad_outputs=g, retain_graph=True)
                    for (x, _), y, g in zip(psets, ys, gs)])
        row(f"{name}_backward_B16_S65536_dp2", st, pub_b)
        del ys, gs
    del psets

    # ---- Sp_SpectralConv2D B=4, 128 -> 32, mode ceil(sqrt(r)) (sp_fno2d.py:10-60) ----
    for r, pub_f, pub_b in ((128, {"V100 exts": 915.2, "V100 torch": 1566.2, "RTX4090 exts": 339.0},
                             {"V100 exts": 1559.5, "RTX4090 exts": 798.3}),
                            (256, {"V100 exts": 3473.6, "V100 torch": 6339.7, "RTX4090 exts": 1829.8},
                             {"V100 exts": 6302.1, "RTX4090 exts": 4226.6}),
                            (512, {"V100 exts": 12688.2, "V100 torch": 30378.5, "RTX4090 exts": 8411.6},
                             {"V100 exts": 24072.0, "RTX4090 exts": 17683.2})):
        mode = math.ceil(math.sqrt(r))
        torch.manual_seed(0)
        layer = L.Sp_SpectralConv2D(128, 32, mode, 0.0, "silu").to(dev)
        nb = 4 * r * r * (128 + 32) * 4
        xs = [ru(4, r, r, 128, requires_grad=True) for _ in range(nsets(nb))]
        with torch.no_grad():
            st = timed([lambda x=x: layer(x) for x in xs])
        row(f"spectral_conv2d_forward_B4_128to32_r{r}_m{mode}", st, pub_f, GBps=round(nb / st["median_us"] / 1e3, 1))
        st = timed([lambda x=x: layer(x) for x in xs])
        row(f"spectral_conv2d_forward_grad_enabled_B4_128to32_r{r}_m{mode}", st, pub_f)
        ys = [layer(x) for x in xs[:2]]
        gs = [torch.rand_like(y) for y in ys]
        st = timed([lambda x=x, y=y, g=g: torch.autograd.grad(outputs=y, inputs=x, grad_outputs=g, retain_graph=True)
                    for x, y, g in zip(xs, ys, gs)])
        row(f"spectral_conv2d_backward_B4_128to32_r{r}_m{mode}", st, pub_b)
        del xs, ys, gs, layer

    # ---- model parts and the whole model at the reference's timing configuration (sp_darcy_breakdown.py:19-40,
    # sp_darcy_ablation.py:23-70): yaml defaults, subsample_node 1, subsample_attn 2, modes ceil(sqrt(r)) ----
    def yaml_cfg(R, drops):
        r_attn = int((R - 1) / 2 + 1)
        d = 0.05 if drops else 0.0
        return dict(
            drop_module=0.0, boundary_condition="dirichlet", target_normalizer=SM.UnitNormalizer(),
            resolution_size=M.get_resolution_size(R, r_attn), dim_node=1, dim_hidden=128, drop_downscaler=d,
            acti_downscaler="relu", num_encoder_layer=6, num_head=4, dim_position=2, attn_norm_eps=1e-6,
            drop_encoder_attn=0.0, drop_encoder_attn_fc=d, attn_xavier=0.01, attn_diagonal=0.01, attn_symmetric=False,
            dim_encoder_ffn=256, drop_encoder_ffn=d, acti_encoder_ffn="relu", drop_upscaler=0.0, acti_upscaler="silu",
            num_decoder_layer=2, dim_target=1, dim_spatial_hidden=32, num_frequence_mode=math.ceil(math.sqrt(R)),
            drop_decoder_layer=0.0, acti_decoder_layer="silu"), r_attn

    # six encoder layers, B=4, r=256 -> S=128^2 (sp_darcy_breakdown.py:69-101)
    for drops in (False, True):
        cfg, ra = yaml_cfg(256, drops)
        torch.manual_seed(0)
        layers = torch.nn.ModuleList([L.Sp_EncoderLayer(
            cfg["dim_hidden"], cfg["num_head"], cfg["dim_position"], cfg["attn_norm_eps"], cfg["drop_encoder_attn"],
            cfg["drop_encoder_attn_fc"], cfg["attn_xavier"], cfg["attn_diagonal"], cfg["attn_symmetric"],
            cfg["dim_encoder_ffn"], cfg["drop_encoder_ffn"], cfg["acti_encoder_ffn"]) for _ in range(6)]).to(dev)

        def stack(x, pos):
            for layer in layers:
                x = layer(x, pos)
            return x
        esets = [(ru(4, ra * ra, 128, requires_grad=True), ru(4, ra * ra, 2)) for _ in range(3)]
        tag = "yaml_droprates" if drops else "droprates_0"
        pub = {"V100 exts": 20549.3, "V100 torch": 44660.9, "RTX4090 exts": 10090.0}
        with torch.no_grad():
            st = timed([lambda x=x, p=p: stack(x, p) for x, p in esets])
        row(f"encoder_layers_x6_forward_B4_S16384_dp2_{tag}", st, pub)
        st = timed([lambda x=x, p=p: stack(x, p) for x, p in esets])
        row(f"encoder_layers_x6_forward_grad_enabled_B4_S16384_dp2_{tag}", st, pub)
        ys = [stack(x, p) for x, p in esets[:2]]
        gs = [torch.rand_like(y) for y in ys]
        st = timed([lambda x=x, y=y, g=g: torch.autograd.grad(outputs=y, inputs=x, grad_outputs=g, retain_graph=True)
                    for (x, _), y, g in zip(esets, ys, gs)])
        row(f"encoder_layers_x6_backward_B4_S16384_dp2_{tag}", st, {"V100 exts": 33985.0, "RTX4090 exts": 16881.7})
        del esets, ys, gs, layers

    # decoder regressor (2 spectral blocks, width 32, 16 modes) and the scalers, B=4, r=256
    cfg, ra = yaml_cfg(256, False)
    torch.manual_seed(0)
    reg = SM.Sp_DecoderRegressor(2, 128, 1, 2, 32, cfg["num_frequence_mode"], 0.0, "silu").to(dev)
    rsets = [(ru(4, 256, 256, 128, requires_grad=True), ru(4, 256, 256, 2)) for _ in range(3)]
    with torch.no_grad():
        st = timed([lambda x=x, g=g: reg(x, grid=g) for x, g in rsets])
    row("decoder_regressor_forward_B4_r256", st, {"V100 exts": 7928.4, "V100 torch": 9361.6, "RTX4090 exts": 2774.6})
    st = timed([lambda x=x, g=g: reg(x, grid=g) for x, g in rsets])
    row("decoder_regressor_forward_grad_enabled_B4_r256", st, {"V100 exts": 7928.4, "RTX4090 exts": 2774.6})
    del rsets, reg
    for drops in (False, True):
        cfg, ra = yaml_cfg(256, drops)
        tag = "yaml_droprates" if drops else "droprates_0"
        down = M.DownScaler2D(cfg["resolution_size"], 1, 128, cfg["drop_downscaler"], "relu").to(dev)
        dsets = [ru(4, 256, 256, 1) for _ in range(3)]
        with torch.no_grad():
            st = timed([lambda x=x: down(x) for x in dsets])
        row(f"down_scaler_forward_B4_r256_{tag}", st, {"V100": 5027.1, "RTX4090": 2457.2})
        del down, dsets
    up = M.UpScaler2D(cfg["resolution_size"], 128, 128, 0.0, "silu").to(dev)
    usets = [ru(4, ra, ra, 128) for _ in range(4)]
    with torch.no_grad():
        st = timed([lambda x=x: up(x) for x in usets])
    row("up_scaler_forward_B4_r256", st, {"V100": 3204.6, "RTX4090": 1387.5})
    del up, usets

    # whole model, B=4: inference forward (sp_darcy_ablation.py:308-314 times forward + the validation metric) and
    # one training step (forward, loss, backward, gradient clipping, Adam; :294-306) with a relative L2 loss
    for R, pub_valid, pub_train in ((128, {"V100 V4": 10500.0, "V100 V0": 16700.0, "RTX4090 V4": 3900.0},
                                     {"V100 V4": 29700.0, "RTX4090 V4": 12300.0}),
                                    (256, {"V100 V4": 37600.0, "V100 V0": 63800.0, "RTX4090 V4": 17100.0},
                                     {"V100 V4": 104600.0, "RTX4090 V4": 50600.0}),
                                    (512, {"V100 V4": 147600.0, "V100 V0": 256200.0, "RTX4090 V4": 74600.0},
                                     {"V100 V4": 394900.0, "RTX4090 V4": 210900.0})):
        for drops in (False, True):
            cfg, ra = yaml_cfg(R, drops)
            tag = "yaml_droprates" if drops else "droprates_0"
            torch.manual_seed(0)
            model = SM.Sp_GalerkinTransformer2D(cfg).to(dev)
            msets = [(ru(4, R, R, 1), ru(4, ra, ra, 2), ru(4, R, R, 2), ru(4, R, R, 1)) for _ in range(3)]

            def valid(node, position, grid, target):
                with torch.no_grad():
                    pred = model(node, position, grid)
                    return ((pred - target) ** 2).mean(dim=(1, 2, 3)).sqrt().mean()
            st = timed([lambda t=t: valid(*t) for t in msets])
            row(f"model_inference_B4_r{R}_{tag}", st, pub_valid,
                samples_per_s=round(4 / st["median_us"] * 1e6, 1))
            del model
        # training step at the yaml's drop rates
        cfg, ra = yaml_cfg(R, True)
        torch.manual_seed(0)
        model = SM.Sp_GalerkinTransformer2D(cfg).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=1e-3)

        def train(node, position, grid, target):
            opt.zero_grad(set_to_none=True)
            pred = model(node, position, grid)
            loss = (((pred - target) ** 2).sum(dim=(1, 2, 3)) / (target ** 2).sum(dim=(1, 2, 3))).sqrt().mean()
            loss.backward()
            torch.nn.utils.clip_grad_norm_(model.parameters(), 0.999)
            opt.step()
            return loss
        st = timed([lambda t=t: train(*t) for t in msets], n=6 if quick else 9, warm=2)
        row(f"model_training_step_B4_r{R}_yaml_droprates", st, pub_train,
            note="relative L2 loss instead of the reference's weighted H1 loss with its regulariser")
        del model, opt, msets
    return out


def recorded_pass_traffic():
    """HBM bytes per launch of the K/V pass and the Q pass from the committed rocprofv3 counter summary (FETCH_SIZE
    and WRITE_SIZE runs, scaled by a copy kernel of known size), {} when the summary is not there.  Counters need
    runs of their own, so these are recorded figures for the same kernels and shape, not live readings."""
    import re
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "fused_attention_B8_S44521_hbm_traffic.md")
    try:
        text = open(path).read()
    except OSError:
        return {}
    found = {}
    for name in ("K/V pass", "Q pass"):
        m = re.search(r"^\| " + re.escape(name) + r" \| ([\d ]+) KiB[^|]*\|[^|]*\| ([\d ]+) KiB", text, re.M)
        if m:
            read_kib, write_kib = (int(g.replace(" ", "")) for g in m.groups())
            found[name] = (read_kib + write_kib) * 1024
    return found


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--input-sets", type=int, default=3,
                    help="independent (Q, K, V) sets the timed steps rotate through")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--spinup", type=int, default=300,
                    help="untimed steps of the same call before the warm-up steps, so that the GPU's clocks have "
                         "settled when the timed steps run (echoed in the output; the step time of the plain "
                         "--warmup/--steps sequence on the GPU as it was found is reported beside it)")
    ap.add_argument("--only", choices=["kernels", "darcy", "published"], default=None,
                    help="profiling aid: run only the per-kernel table (every operator of the path at its benchmark "
                         "shape), only a few end-to-end Darcy forwards, or only the reference's published workloads, "
                         "and print that part as JSON")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    from spgt_amd.extension.bind import galerkin_attention as ga

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP path has no CPU fallback)")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.only == "kernels":
        if args.calibrate_copy:
            src = torch.empty(256 * 1024 * 1024 // 4, device=dev).normal_()
            dst = torch.empty_like(src)
            for _ in range(5):
                dst.copy_(src)  # reads 256 MiB, writes 256 MiB
            torch.cuda.synchronize()
            del src, dst
        print(json.dumps({"kernel_rooflines": kernel_rooflines(dev, use_graph=False)}))
        return
    if args.only == "published":
        print(json.dumps({"reference_published_shapes": reference_published_shapes(dev, quick=args.steps < 50)}))
        return
    if args.only == "darcy":
        print(json.dumps({"darcy_inference": darcy_bench(dev, with_cpu=False, steps=max(1, min(args.steps, 20)),
                                                         graph=False)}))
        return

    B, S, H, dp = 8, 44521, 4, 0
    g = torch.Generator(device=dev).manual_seed(0)
    # Independent (Q, K, V) sets visited in turn: one set is 547 MB, so when a set comes round again
    # 1.6 GB of other inputs and outputs have passed through the 256 MB last-level cache.
    n_sets = max(1, args.input_sets)
    sets = [tuple(torch.randn(B, S, H * 32, device=dev, generator=g) for _ in range(3)) for _ in range(n_sets)]
    one, zero = torch.ones(H, 32, device=dev), torch.zeros(H, 32, device=dev)
    nbytes = 4 * B * H * 32 * S * 4

    # A step goes through the C ABI directly, as a compiled caller would: outputs (one per input set, so that no
    # step overwrites lines the previous one left in the cache), K^T V / S and the workspace are allocated once.
    import ctypes
    from spgt_amd import _lib
    lib = _lib.load()
    outs = [torch.empty(B, S, H * 32, device=dev) for _ in range(n_sets)]
    ktv = torch.empty(B, H, 32, 32, device=dev)
    ws_bytes = lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dp)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    call_args = [(vp(q), vp(k), vp(v), H * 32, None, vp(one), vp(zero), vp(one), vp(zero), 1e-6, vp(o), vp(ktv), vp(ws),
                  ws_bytes, B, S, H, dp, stream) for (q, k, v), o in zip(sets, outs)]
    fused = lib.spgt_galerkin_attention_fused_forward

    def step(i):
        if fused(*call_args[i % n_sets]) != 0:
            raise RuntimeError(_lib.last_error())

    def wall_ms(fn):
        for i in range(args.warmup):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    # First the caller's sequence as it stands, on the GPU as it was found: `warmup` untimed steps, `steps` timed.
    # The clocks of an idle GPU need tens of milliseconds of load to settle (20 timed steps after 5 warm-up steps
    # read 7-9 % longer than the same steps after 100), so the figure that `value` is computed from is taken
    # after `--spinup` further untimed steps of the same call plus the warm-up again; both are reported.
    ms_without_spinup = wall_ms(step)
    spinup_steps = max(0, args.spinup)
    for i in range(spinup_steps):
        step(i)
    torch.cuda.synchronize()
    ms_per_step = wall_ms(step) if spinup_steps else ms_without_spinup  # exactly `steps` calls, operands rotated
    value = nbytes / (ms_per_step * 1e-3) / 1e9
    same_ms = wall_ms(lambda i: step(0))  # every step on one set (Q and out fit the last-level cache)
    binding_ms = wall_ms(lambda i: ga.galerkin_attention_fused(*sets[i % n_sets], None, one, zero, one, zero, 1e-6,
                                                               H, dp))  # the Python operator, allocating its output
    # host time per step without the GPU in the way: how far the launch rate is from bounding the loop
    t0 = time.perf_counter()
    for i in range(20):
        step(i)
    host_us = (time.perf_counter() - t0) / 20 * 1e6
    torch.cuda.synchronize()

    # per-call and per-launch durations of the same rotated sequence: HIP events on the launch stream
    # around every launch, calls back to back, one synchronisation at the end
    n_prof = max(30, min(args.steps, 400))
    ga.gexts.galerkin_attention_fused_profile(sets, None, one, zero, one, zero, 1e-6, H, dp, 10)
    stages = ga.gexts.galerkin_attention_fused_profile(sets, None, one, zero, one, zero, 1e-6, H, dp, n_prof)

    def dist(vals):
        vs = sorted(vals)
        pick = lambda f: vs[min(len(vs) - 1, int(f * len(vs)))]
        return {"median": round(pick(0.5) * 1e3, 2), "p10": round(pick(0.1) * 1e3, 2), "p90": round(pick(0.9) * 1e3, 2)}

    kv = dist([st[0] for st in stages])
    kv_bytes = 2 * B * H * 32 * S * 4  # K and V read once; partial tiles are not counted
    q_bytes = 2 * B * H * 32 * S * 4   # Q read once, out written once
    qd = dist([st[2] for st in stages])
    # the kernel that takes the largest share of a call is the Q pass (rocprofv3: 51 % of kernel time)
    achieved = q_bytes / (qd["median"] * 1e-6) / 1e9
    call = dist([sum(st) for st in stages])
    traffic = recorded_pass_traffic()
    roofline = {
        "bound": "hbm", "kernel": "qm_apply_tm<0,2>", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
        "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic.get("Q pass"),
        "traffic_source": "recorded: rocprofv3 FETCH_SIZE + WRITE_SIZE summary under profiles/ for this kernel and "
                          "shape (counters need runs of their own), not a reading of this run",
        "kernel_us": qd["median"], "kernel_us_p10_p90": [qd["p10"], qd["p90"]], "algorithmic_bytes": q_bytes,
        "timing": f"HIP events around each launch, {n_prof} calls back to back over {n_sets} rotated input and "
                  "output sets, median",
        "stages_us": {"kv_pass": kv, "tile_reduce": dist([st[1] for st in stages]), "q_pass": qd, "call": call},
        "kv_pass": {"kernel": "ktv_ln_partial_tm<0,4,4>", "algorithmic_bytes": kv_bytes,
                    "GBps": round(kv_bytes / (kv["median"] * 1e-6) / 1e9, 1),
                    "frac": round(kv_bytes / (kv["median"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                    "traffic": traffic.get("K/V pass")},
        "whole_call": {"algorithmic_bytes": nbytes, "GBps": round(nbytes / (call["median"] * 1e-6) / 1e9, 1),
                       "frac": round(nbytes / (call["median"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)},
    }

    extra = {}
    if args.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024 // 4, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)  # vectorized elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        extra["calibrate_copy_bytes_each_way"] = src.numel() * 4
        del src, dst
    if not args.no_extra:
        def timed(fn, n=50, warm=5):
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n

        # what this part copies at: torch's elementwise copy of the Q pass's bytes (182 MB read, 182 MB written),
        # sources and destinations rotated like the benchmark's inputs
        dsts = [torch.empty_like(sets[0][0]) for _ in range(2)]
        cnt = [0]

        def plain_copy():
            cnt[0] += 1
            dsts[cnt[0] % 2].copy_(sets[cnt[0] % n_sets][cnt[0] % 3])

        ms = timed(plain_copy)
        extra["plain_copy_182MB_rotated"] = {"ms": round(ms, 4), "GB/s": round(q_bytes / ms / 1e6, 1)}
        del dsts
        Qf, Kf, Vf = (torch.randn(B, H, 32, S, device=dev, generator=g) for _ in range(3))
        ms = timed(lambda: ga.multihead_galerkin_attention_cccr_cuda(Qf, Kf, Vf))
        extra["attention_cccr_d32"] = {"ms": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1)}
        del Qf, Kf, Vf
        g1 = torch.Generator(device=dev).manual_seed(1)
        A = torch.randn(32, 32, S, device=dev, generator=g1)
        Bm = torch.randn(32, S, 32, device=dev, generator=g1)
        c2_bytes = 2 * 32 * 32 * S * 4 + 32 * 32 * 32 * 4
        ms = timed(lambda: ga.batched_skinny_gemm(A, Bm, 1.0))
        extra["config2_split_k_gemm"] = {"ms": round(ms, 4), "GB/s": round(c2_bytes / ms / 1e6, 1)}
        ms = timed(lambda: torch.matmul(A, Bm))
        extra["config2_torch_matmul"] = {"ms": round(ms, 4), "GB/s": round(c2_bytes / ms / 1e6, 1)}
        del A, Bm
        extra["kernel_rooflines"] = kernel_rooflines(dev)
        extra["reference_published_shapes"] = reference_published_shapes(dev, quick=True)
        extra["darcy_inference"] = darcy_bench(dev, with_cpu=not args.no_cpu_baseline)
        extra["encoder_stack_config3"] = encoder_stack_bench(dev, with_cpu=not args.no_cpu_baseline)
        extra["fno_stack_config4"] = fno_stack_bench(dev, with_cpu=not args.no_cpu_baseline)

    result = {
        "metric": "galerkin_attn_hbm_gbps", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "untimed_steps_before_timing": 2 * args.warmup + spinup_steps + args.steps
        if spinup_steps else args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fused Galerkin attention core (LayerNorm K,V + K^T V/S + Q(K^T V/S)), "
                               "B=8 S=44521 d_model=128 heads=4 dp=0, token-major projections resident in HBM",
                   "algorithmic_bytes_per_step": nbytes, "hbm_frac_of_8TBps": round(value / HBM_PEAK_GBPS, 4),
                   "input_sets_rotated": n_sets,
                   "untimed_spinup_steps_before_warmup": spinup_steps,
                   "ms_per_step_without_spinup": round(ms_without_spinup, 4),
                   "GBps_without_spinup": round(nbytes / ms_without_spinup / 1e6, 1),
                   "hbm_frac_without_spinup": round(nbytes / ms_without_spinup / 1e6 / HBM_PEAK_GBPS, 4),
                   "ms_per_step_one_input_set": round(same_ms, 4),
                   "GBps_one_input_set": round(nbytes / same_ms / 1e6, 1),
                   "ms_per_step_python_operator": round(binding_ms, 4),
                   "host_us_per_step_issue": round(host_us, 1)},
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(B, S, H, 0),
        "extra": extra,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
