"""Parity of the HIP attention kernels (through the C ABI) with the CPU oracle.

Tolerance: max|y - y_ref| / max|y_ref| <= 1e-4 against the oracle evaluated in
fp64 on the same fp32 inputs (the north-star bound); in practice the kernels
sit near 1e-6.
"""
import ctypes

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


def heads_token_major(t, H):
    """[B, H, S, d] -> [B, S, H*d]"""
    B, _, S, d = t.shape
    return t.permute(0, 2, 1, 3).reshape(B, S, H * d)


def fused_reference(q, k, v, pos, gK, bK, gV, bV, eps, H, dp, dtype=torch.float64):
    """Oracle on raw projections: identity projection weights, so the oracle's
    LayerNorm/concat/matmul chain runs on exactly the kernel's inputs."""
    B, S, C = q.shape
    c = lambda t: t.to(dtype)
    eye, zero = torch.eye(C, dtype=dtype), torch.zeros(C, dtype=dtype)
    posd = c(pos) if dp else torch.zeros(B, S, 0, dtype=dtype)
    Q = O.project_heads(c(q), eye, zero, posd, H, 32)
    K = O.project_layernorm_heads(c(k), eye, zero, c(gK), c(bK), posd, eps, H, 32)
    V = O.project_layernorm_heads(c(v), eye, zero, c(gV), c(bV), posd, eps, H, 32)
    out = heads_token_major(O.galerkin_attention(Q, K, V), H)
    return out, O.attention_ktv(K, V)


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,S,H", [(1, 1, 4), (2, 50, 4), (1, 777, 4), (3, 4099, 4), (2, 1000, 8),
                                   # long sequences: the K/V pass runs 1024-thread workgroups whose four token
                                   # sub-ranges per head meet in LDS; ragged last chunks, two head groups
                                   (2, 150001, 4), (1, 140003, 8)])
def test_fused_attention_vs_oracle(gpu, dp, B, S, H):
    C = H * 32
    q, k, v = rnd(B, S, C, seed=1), rnd(B, S, C, seed=2) * 1.7 + 0.3, rnd(B, S, C, seed=3) * 0.6 - 0.2
    pos = torch.rand(B, S, 2, generator=torch.Generator().manual_seed(4))
    gK, bK, gV, bV = (1 + 0.3 * rnd(H, 32, seed=5)), 0.2 * rnd(H, 32, seed=6), (1 + 0.3 * rnd(H, 32, seed=7)), \
        0.2 * rnd(H, 32, seed=8)
    eps = 1e-6
    want, want_ktv = fused_reference(q, k, v, pos, gK, bK, gV, bV, eps, H, dp)
    d = lambda t: t.to(gpu)
    out, ktv = ga.galerkin_attention_fused(d(q), d(k), d(v), d(pos) if dp else None, d(gK), d(bK), d(gV), d(bV), eps,
                                           H, dp, return_ktv=True)
    torch.cuda.synchronize()
    assert out.shape == (B, S, H * (dp + 32))
    assert max_rel(ktv.cpu().double(), want_ktv) < TOL
    assert max_rel(out.cpu().double(), want) < TOL


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,S,H", [(1, 1, 4), (2, 50, 4), (3, 4099, 4), (2, 1000, 8)])
def test_attention_folded_into_projection(gpu, dp, B, S, H):
    """K/V pass alone, and the fold of K~^T V~ / S into the output projection: the attention output times fc_layer's
    weight (network/sp_layer.py:64-75) must equal Q times the folded weight plus the position rows' share, by
    associativity; against the oracle in float64."""
    C = H * 32
    D = dp + 32
    q, k, v = rnd(B, S, C, seed=1), rnd(B, S, C, seed=2) * 1.7 + 0.3, rnd(B, S, C, seed=3) * 0.6 - 0.2
    pos = torch.rand(B, S, 2, generator=torch.Generator().manual_seed(4))
    gK, bK, gV, bV = (1 + 0.3 * rnd(H, 32, seed=5)), 0.2 * rnd(H, 32, seed=6), (1 + 0.3 * rnd(H, 32, seed=7)), \
        0.2 * rnd(H, 32, seed=8)
    eps = 1e-6
    want_out, want_ktv = fused_reference(q, k, v, pos, gK, bK, gV, bV, eps, H, dp)
    d = lambda t: t.to(gpu)
    ktv = ga.galerkin_attention_ktv(d(k), d(v), d(pos) if dp else None, d(gK), d(bK), d(gV), d(bV), eps, H, dp)
    _, ktv_full = ga.galerkin_attention_fused(d(q), d(k), d(v), d(pos) if dp else None, d(gK), d(bK), d(gV), d(bV),
                                              eps, H, dp, return_ktv=True)
    assert torch.equal(ktv, ktv_full)  # the same two launches
    assert max_rel(ktv.cpu().double(), want_ktv) < TOL
    N = 128
    wfc = rnd(H * D, N, seed=9) / 8
    folded, folded_pos = ga.fold_ktv_into_fc(ktv, d(wfc), dp)
    assert folded.shape == (B, H * 32, N) and (folded_pos is None) == (dp == 0)
    got = torch.einsum("bsc,bcn->bsn", q.double(), folded.cpu().double())
    if dp:
        assert folded_pos.shape == (B, dp, N)
        got = got + torch.einsum("bsp,bpn->bsn", pos.double(), folded_pos.cpu().double())
    want = want_out @ wfc.double()
    assert max_rel(got, want) < TOL
    # the folded weight itself: M_h Wfc_h, feature rows per head and position rows summed over the heads
    m = ktv.cpu().double()
    w = wfc.double().view(H, D, N)
    full = torch.einsum("bhij,hjn->bhin", m, w)
    assert max_rel(folded.cpu().double(), full[:, :, dp:].reshape(B, H * 32, N)) < 1e-5
    if dp:
        assert max_rel(folded_pos.cpu().double(), full[:, :, :dp].sum(1)) < 1e-5


def test_fused_attention_strided_qkv(gpu):
    """Q, K, V as column slices of one [B, S, 384] projection output."""
    B, S, H = 2, 333, 4
    qkv = rnd(B, S, 3 * H * 32, seed=11)
    gK, bK, gV, bV = (1 + 0.3 * rnd(H, 32, seed=5)), 0.2 * rnd(H, 32, seed=6), (1 + 0.3 * rnd(H, 32, seed=7)), \
        0.2 * rnd(H, 32, seed=8)
    q, k, v = qkv[..., :128], qkv[..., 128:256], qkv[..., 256:]
    want, _ = fused_reference(q.contiguous(), k.contiguous(), v.contiguous(), None, gK, bK, gV, bV, 1e-5, H, 0)
    g = qkv.to(gpu)
    out = ga.galerkin_attention_fused(g[..., :128], g[..., 128:256], g[..., 256:], None, gK.to(gpu), bK.to(gpu),
                                      gV.to(gpu), bV.to(gpu), 1e-5, H, 0)
    assert max_rel(out.cpu().double(), want) < TOL


@pytest.mark.parametrize("dp", [0, 2])
def test_fused_attention_golden(gpu, dp):
    """From the reference module's parameters and input to its pre-fc attention
    output: projections by torch on the GPU, everything else by the fused kernel."""
    p, i, _, meta = load_golden(f"attention_dp{dp}")
    _, pieces, want, _ = load_golden(f"attention_pieces_dp{dp}")
    H, eps = int(meta["num_head"]), float(meta["norm_eps"])
    x = i["x"].to(gpu)
    proj = lambda n: torch.nn.functional.linear(x, p["weight_" + n].to(gpu), p["bias_" + n].to(gpu))
    d = lambda t: t.to(gpu).contiguous()
    out = ga.galerkin_attention_fused(proj("Q"), proj("K"), proj("V"), d(i["position"]) if dp else None,
                                      d(p["ln_weight_K"]), d(p["ln_bias_K"]), d(p["ln_weight_V"]), d(p["ln_bias_V"]),
                                      eps, H, dp)
    assert max_rel(out.cpu(), heads_token_major(want, H)) < TOL


@pytest.mark.parametrize("d", [32, 34])
@pytest.mark.parametrize("B,H,S", [(1, 1, 1), (2, 4, 50), (1, 4, 777), (2, 3, 4099), (1, 2, 12345)])
def test_attention_cccr_vs_oracle(gpu, d, B, H, S):
    Q, K, V = rnd(B, H, d, S, seed=21), rnd(B, H, d, S, seed=22), rnd(B, H, d, S, seed=23)
    want = O.op_attention_cccr(Q.double(), K.double(), V.double())
    got = ga.multihead_galerkin_attention_cccr_cuda(Q.to(gpu), K.to(gpu), V.to(gpu))
    assert got.shape == (B, H, S, d)
    assert max_rel(got.cpu().double(), want) < TOL


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_cccr_golden(gpu, dp):
    _, i, want, _ = load_golden(f"attention_pieces_dp{dp}")
    t = lambda a: a.transpose(-2, -1).contiguous().to(gpu)
    got = ga.multihead_galerkin_attention_cccr_cuda(t(i["Q"]), t(i["K"]), t(i["V"]))
    assert max_rel(got.cpu(), want) < TOL


def test_attention_cccr_special_cases(gpu):
    S, d = 4096, 32
    ones = torch.ones(1, 4, d, S, device=gpu)
    got = ga.multihead_galerkin_attention_cccr_cuda(ones, ones, ones)
    assert torch.allclose(got, torch.full_like(got, float(d)), rtol=1e-6, atol=0)
    Kq, _ = torch.linalg.qr(rnd(S, d, seed=31).double())
    K = Kq.t().float()[None, None].contiguous().to(gpu)
    Q = rnd(1, 1, d, S, seed=32).to(gpu)
    got = ga.multihead_galerkin_attention_cccr_cuda(Q, K, K)
    assert max_rel(got, Q.transpose(-2, -1) / S) < 1e-5


ORDERS = ["RRR", "RRC", "RCR", "RCC", "CRR", "CRC", "CCR", "CCC"]


def skinny_gemm_any_order(A, B, alpha, order):
    """A [b, M, K], B [b, K, N] logical; stores them in `order`, calls the C ABI, returns logical C."""
    lib = _lib.load()
    b, M, K = A.shape
    N = B.shape[-1]
    a_mem = A.contiguous() if order[0] == "R" else A.transpose(1, 2).contiguous()
    b_mem = B.contiguous() if order[1] == "R" else B.transpose(1, 2).contiguous()
    c_mem = torch.full((b, M * N), float("nan"), device=A.device)
    ws = _lib.workspace(lib.spgt_batched_skinny_gemm_workspace_bytes(M, N, K, b), A)
    _lib.check(lib.spgt_batched_skinny_gemm(
        _lib.ptr(a_mem), _lib.ptr(b_mem), _lib.ptr(c_mem), alpha, M, N, K, M * K, K * N, M * N,
        ga.GEMM_ORDER[order], b, _lib.ptr(ws), ws.numel(), _lib.stream_of(A)))
    return c_mem.view(b, M, N) if order[2] == "R" else c_mem.view(b, N, M).transpose(1, 2)


@pytest.mark.parametrize("order", ORDERS)
def test_skinny_gemm_orders_and_shapes(gpu, order):
    shapes = [(1, 1, 1, 1), (2, 32, 32, 64), (3, 5, 7, 63), (2, 33, 31, 65), (1, 40, 17, 1000), (2, 32, 32, 5000),
              (1, 3, 64, 129), (2, 34, 34, 4097)]
    for n, (b, M, N, K) in enumerate(shapes):
        A, B = rnd(b, M, K, seed=40 + n), rnd(b, K, N, seed=60 + n)
        want = O.op_batched_skinny_gemm(A.double(), B.double(), 0.5)
        got = skinny_gemm_any_order(A.to(gpu), B.to(gpu), 0.5, order)
        assert not torch.isnan(got).any(), (order, b, M, N, K)
        assert max_rel(got.cpu().double(), want) < 1e-5, (order, b, M, N, K)


def small_k_gemm_any_order(A, B, alpha, order):
    """As skinny_gemm_any_order through spgt_batched_small_k_gemm (one launch, no workspace)."""
    lib = _lib.load()
    b, M, K = A.shape
    N = B.shape[-1]
    a_mem = A.contiguous() if order[0] == "R" else A.transpose(1, 2).contiguous()
    b_mem = B.contiguous() if order[1] == "R" else B.transpose(1, 2).contiguous()
    c_mem = torch.full((b, M * N), float("nan"), device=A.device)
    _lib.check(lib.spgt_batched_small_k_gemm(
        _lib.ptr(a_mem), _lib.ptr(b_mem), _lib.ptr(c_mem), alpha, M, N, K, M * K, K * N, M * N,
        ga.GEMM_ORDER[order], b, _lib.stream_of(A)))
    return c_mem.view(b, M, N) if order[2] == "R" else c_mem.view(b, N, M).transpose(1, 2)


@pytest.mark.parametrize("order", ORDERS)
def test_small_k_gemm_orders_and_shapes(gpu, order):
    """The reference's small-K batched GEMM (extension/native/sgemm_32x32.cu:683-710) in all eight operand orders:
    long M with K = d (the Q M product), long N (the backward's products), ragged tiles, K beyond one step."""
    shapes = [(1, 1, 1, 1), (2, 5041, 34, 34), (3, 32, 777, 32), (2, 100, 65, 48), (1, 33, 31, 7), (2, 64, 64, 130),
              (4, 1000, 32, 32)]
    for n, (b, M, N, K) in enumerate(shapes):
        A, B = rnd(b, M, K, seed=140 + n), rnd(b, K, N, seed=160 + n)
        want = O.op_batched_skinny_gemm(A.double(), B.double(), 0.25)
        got = small_k_gemm_any_order(A.to(gpu), B.to(gpu), 0.25, order)
        assert not torch.isnan(got).any(), (order, b, M, N, K)
        assert max_rel(got.cpu().double(), want) < 1e-5, (order, b, M, N, K)
        again = small_k_gemm_any_order(A.to(gpu), B.to(gpu), 0.25, order)
        assert torch.equal(got, again)


def test_skinny_gemm_every_k(gpu):
    """K around every tile/step boundary (the reference's split heuristic can start a split beyond K)."""
    for K in list(range(1, 140)) + [255, 256, 257, 4095, 4096, 4097, 4999]:
        A, B = rnd(2, 32, K, seed=K), rnd(2, K, 32, seed=K + 7)
        got = ga.batched_skinny_gemm(A.to(gpu), B.to(gpu), 1.0)
        assert max_rel(got.cpu().double(), A.double() @ B.double()) < 1e-5, K


def test_skinny_gemm_leading_dims_and_determinism(gpu):
    A, B = rnd(2, 3, 32, 3001, seed=71).to(gpu), rnd(2, 3, 3001, 32, seed=72).to(gpu)
    c1 = ga.batched_skinny_gemm(A, B, 1.0 / 3001)
    c2 = ga.batched_skinny_gemm(A, B, 1.0 / 3001)
    assert c1.shape == (2, 3, 32, 32)
    assert torch.equal(c1, c2)
    assert max_rel(c1.cpu().double(), (A.cpu().double() @ B.cpu().double()) / 3001) < 1e-5


def test_attention_determinism(gpu):
    B, S, H = 2, 5000, 4
    q, k, v = rnd(B, S, 128, seed=81).to(gpu), rnd(B, S, 128, seed=82).to(gpu), rnd(B, S, 128, seed=83).to(gpu)
    one, zero = torch.ones(H, 32, device=gpu), torch.zeros(H, 32, device=gpu)
    a = ga.galerkin_attention_fused(q, k, v, None, one, zero, one, zero, 1e-6, H, 0)
    b = ga.galerkin_attention_fused(q, k, v, None, one, zero, one, zero, 1e-6, H, 0)
    assert torch.equal(a, b)


def test_full_size_properties(gpu):
    """B=8, S=44521, 4 heads (the benchmark shape): size-independent checks."""
    B, S, H = 8, 44521, 4
    gen = torch.Generator(device=gpu).manual_seed(5)
    q = torch.randn(B, S, 128, device=gpu, generator=gen)
    k = torch.randn(B, S, 128, device=gpu, generator=gen)
    v = torch.randn(B, S, 128, device=gpu, generator=gen)
    one, zero = torch.ones(H, 32, device=gpu), torch.zeros(H, 32, device=gpu)
    # gamma = 0, beta = 1: K' = V' = 1 exactly, so K'^T V'/S = 1 and out = row sums of Q per head
    out, ktv = ga.galerkin_attention_fused(q, k, v, None, zero, one, zero, one, 1e-6, H, 0, return_ktv=True)
    assert torch.allclose(ktv, torch.ones_like(ktv), rtol=1e-6, atol=0)
    rowsum = q.view(B, S, H, 32).double().sum(-1, keepdim=True).expand(-1, -1, -1, 32).reshape(B, S, 128)
    assert max_rel(out.double(), rowsum) < 1e-5
    # linear in Q
    out1, ktv1 = ga.galerkin_attention_fused(q, k, v, None, one, zero, one, zero, 1e-6, H, 0, return_ktv=True)
    out2 = ga.galerkin_attention_fused(2 * q, k, v, None, one, zero, one, zero, 1e-6, H, 0)
    assert torch.equal(out2, 2 * out1)
    # against torch's own GPU ops at full size (fp32 both sides)
    kn = torch.nn.functional.layer_norm(k.view(B, S, H, 32), (32,), eps=1e-6)
    vn = torch.nn.functional.layer_norm(v.view(B, S, H, 32), (32,), eps=1e-6)
    m = torch.einsum("bshi,bshj->bhij", kn.double(), vn.double()) / S
    assert max_rel(ktv1.double(), m) < TOL
    ref = torch.einsum("bshi,bhij->bshj", q.view(B, S, H, 32).double(), m).reshape(B, S, 128)
    assert max_rel(out1.double(), ref) < TOL
    # and the oracle itself on one batch entry
    want, _ = fused_reference(q[:1].cpu(), k[:1].cpu(), v[:1].cpu(), None, one.cpu(), zero.cpu(), one.cpu(),
                              zero.cpu(), 1e-6, H, 0, dtype=torch.float32)
    assert max_rel(out1[:1].cpu(), want) < TOL


def test_config2_split_k(gpu):
    """32 problems of K^T[32 x 44521] . V[44521 x 32], N(0,1), seed 1."""
    g = torch.Generator().manual_seed(1)
    A = torch.randn(32, 32, 44521, generator=g)
    B = torch.randn(32, 44521, 32, generator=g)
    got = ga.batched_skinny_gemm(A.to(gpu), B.to(gpu), 1.0)
    want = A.double() @ B.double()
    assert max_rel(got.cpu().double(), want) < 1e-5


def test_argument_validation(gpu):
    lib = _lib.load()
    q = torch.zeros(1, 4, 33, 16, device=gpu)
    with pytest.raises(ValueError):
        ga.multihead_galerkin_attention_cccr_cuda(q, q, q)
    q = torch.zeros(1, 4, 32, 16, device=gpu)
    ws = torch.empty(16, dtype=torch.uint8, device=gpu)
    out = torch.empty(1, 4, 16, 32, device=gpu)
    rc = lib.spgt_galerkin_attention_cccr_forward(_lib.ptr(q), _lib.ptr(q), _lib.ptr(q), _lib.ptr(out), _lib.ptr(ws),
                                                  16, 1, 4, 32, 16, None)
    assert rc == -2 and "workspace" in _lib.last_error()
    with pytest.raises(TypeError):
        ga.batched_skinny_gemm(q.double(), q.double())
