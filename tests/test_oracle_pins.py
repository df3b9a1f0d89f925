"""Pins for the oracle helpers that the GPU tests, smoke() and the CPU baseline
lean on: each is checked against the reference's own golden vectors, a
brute-force loop, or a number worked out by hand - never against its own formula."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import load_golden, max_rel
from oracle import spgt_oracle as O

TOL = 2e-6


def rnd(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_core_token_major_vs_reference_golden(dp):
    """Linear projections -> attention_core_token_major -> fc_layer must reproduce the
    reference module's output (GalerkinAttention.forward, network/layer.py:67-93)."""
    p, i, out, meta = load_golden(f"attention_dp{dp}")
    x, pos, H, eps = i["x"], i["position"], meta["num_head"], meta["norm_eps"]
    q = F.linear(x, p["weight_Q"], p["bias_Q"])
    k = F.linear(x, p["weight_K"], p["bias_K"])
    v = F.linear(x, p["weight_V"], p["bias_V"])
    core = O.attention_core_token_major(q, k, v, pos, p["ln_weight_K"], p["ln_bias_K"], p["ln_weight_V"],
                                        p["ln_bias_V"], eps, H)
    assert core.shape == (x.shape[0], x.shape[1], H * (dp + 32))
    got = F.linear(core, p["fc_layer.weight"], p["fc_layer.bias"])
    assert max_rel(got, out) < TOL
    # the merged layout is per head [position(dp) | features(32)]: the position
    # columns of the core are Q's position columns times the head's matrix, so
    # swapping two heads' blocks must break the match with the reference
    swapped = core.reshape(*core.shape[:2], H, dp + 32)[:, :, [1, 0, 2, 3]].reshape(core.shape)
    assert max_rel(F.linear(swapped, p["fc_layer.weight"], p["fc_layer.bias"]), out) > 1e-3


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_ktv_vs_reference_golden(dp):
    """Q @ attention_ktv(K, V) must equal the reference's multihead_galerkin_attention
    (network/layer.py:143-152) on the reference's own Q, K, V."""
    _, i, out, _ = load_golden(f"attention_pieces_dp{dp}")
    M = O.attention_ktv(i["K"], i["V"])
    d = i["Q"].shape[-1]
    assert M.shape == (*i["Q"].shape[:2], d, d)
    assert max_rel(i["Q"] @ M, out) < TOL
    # K and V are not interchangeable
    assert max_rel(i["Q"] @ O.attention_ktv(i["V"], i["K"]), out) > 1e-3


def test_attention_ktv_bruteforce():
    B, H, S, d = 2, 3, 8, 5
    K, V = rnd(B, H, S, d, seed=31), rnd(B, H, S, d, seed=32)
    k, v = K.numpy(), V.numpy()
    want = np.zeros((B, H, d, d))
    for b in range(B):
        for h in range(H):
            for i in range(d):
                for j in range(d):
                    acc = 0.0
                    for s in range(S):
                        acc += k[b, h, s, i] * v[b, h, s, j]
                    want[b, h, i, j] = acc / S
    np.testing.assert_allclose(O.attention_ktv(K, V).numpy(), want, rtol=1e-12, atol=1e-13)


def test_attention_core_token_major_bruteforce():
    """Tiny case by loops: heads split in order, LayerNorm per head over its own 32
    features with the head's affine row, position first, heads merged in order."""
    B, S, H, dh, dp, eps = 1, 3, 2, 32, 2, 1e-6
    q, k, v = rnd(B, S, H * dh, seed=33), rnd(B, S, H * dh, seed=34), rnd(B, S, H * dh, seed=35)
    pos = rnd(B, S, dp, seed=36)
    gK, bK, gV, bV = (rnd(H, dh, seed=s) for s in (37, 38, 39, 40))
    got = O.attention_core_token_major(q, k, v, pos, gK, bK, gV, bV, eps, H).numpy()

    def ln(row, g, b):
        mu = sum(row) / dh
        var = sum((t - mu) ** 2 for t in row) / dh
        return [(t - mu) / np.sqrt(var + eps) * g[j] + b[j] for j, t in enumerate(row)]

    d = dp + dh
    want = np.zeros((B, S, H * d))
    for h in range(H):
        Qh = [list(pos[0, s].numpy()) + list(q[0, s, h * dh:(h + 1) * dh].numpy()) for s in range(S)]
        Kh = [list(pos[0, s].numpy()) + ln(k[0, s, h * dh:(h + 1) * dh].numpy(), gK[h].numpy(), bK[h].numpy())
              for s in range(S)]
        Vh = [list(pos[0, s].numpy()) + ln(v[0, s, h * dh:(h + 1) * dh].numpy(), gV[h].numpy(), bV[h].numpy())
              for s in range(S)]
        M = [[sum(Kh[s][a] * Vh[s][c] for s in range(S)) / S for c in range(d)] for a in range(d)]
        for s in range(S):
            for c in range(d):
                want[0, s, h * d + c] = sum(Qh[s][a] * M[a][c] for a in range(d))
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


def test_projection_layernorm_op_invsigma_nonsymmetric_weight():
    """invsigma[b, h, s] = 1/sqrt(var_j(x[b,s,:] @ W[:, h*32+j] + bias) + eps) with W used
    as stored (x @ W, extension/native/multihead_dim32.cu:343-344): explicit loops with a
    weight that is far from symmetric, so W^T in its place fails."""
    B, S, H, dh, dp, eps = 2, 4, 4, 32, 2, 1e-6
    C = H * dh
    x, W, b = rnd(B, S, C, seed=41), rnd(C, C, seed=42), rnd(C, seed=43)
    W = W + 3.0 * torch.triu(torch.ones(C, C, dtype=torch.float64), diagonal=1)
    g, be, pos = rnd(H, dh, seed=44), rnd(H, dh, seed=45), rnd(B, S, dp, seed=46)
    y, inv = O.op_projection_layernorm_rrc(x, W, b, g, be, pos, eps, H, dh)
    assert y.shape == (B, H, dp + dh, S) and inv.shape == (B, H, S)
    xn, Wn, bn = x.numpy(), W.numpy(), b.numpy()
    for bb in range(B):
        for h in range(H):
            for s in range(S):
                row = [sum(xn[bb, s, kk] * Wn[kk, h * dh + j] for kk in range(C)) + bn[h * dh + j]
                       for j in range(dh)]
                mu = sum(row) / dh
                var = sum((t - mu) ** 2 for t in row) / dh
                want_inv = 1.0 / np.sqrt(var + eps)
                assert abs(inv[bb, h, s].item() - want_inv) <= 1e-10 * want_inv
                for j in (0, 13, 31):
                    want = (row[j] - mu) * want_inv * g[h, j].item() + be[h, j].item()
                    assert abs(y[bb, h, dp + j, s].item() - want) < 1e-9
                for c in range(dp):
                    assert y[bb, h, c, s] == pos[bb, s, c]
    # the transposed weight gives something else
    _, inv_t = O.op_projection_layernorm_rrc(x, W.t().contiguous(), b, g, be, pos, eps, H, dh)
    assert (inv_t - inv).abs().max() > 1e-3


def test_gauss_inverse_transform_by_hand():
    """X * (std + eps) + mean (dataset/darcy_dataset.py:30-31), numbers worked by hand."""
    x = torch.tensor([[-2.0, 0.0], [0.5, 4.0]], dtype=torch.float64)
    got = O.gauss_inverse_transform(x, mean=3.0, std=0.25, eps=0.5)
    # std + eps = 0.75: -2*0.75+3 = 1.5, 0+3 = 3, 0.5*0.75+3 = 3.375, 4*0.75+3 = 6
    assert torch.equal(got, torch.tensor([[1.5, 3.0], [3.375, 6.0]], dtype=torch.float64))
    # per-position statistics (what fit(axis=0) produces) broadcast over the batch
    mean = torch.tensor([1.0, -1.0], dtype=torch.float64)
    std = torch.tensor([1.0, 3.0], dtype=torch.float64)
    got = O.gauss_inverse_transform(x, mean=mean, std=std, eps=1.0)
    assert torch.equal(got, torch.tensor([[-3.0, -1.0], [2.0, 15.0]], dtype=torch.float64))
    # it is the inverse of (X - mean) / (std + eps)  (darcy_dataset.py:27-28)
    z = (x - mean) / (std + 1e-5)
    torch.testing.assert_close(O.gauss_inverse_transform(z, mean, std, 1e-5), x, rtol=1e-14, atol=1e-14)
    # defaults: mean 0, std 1, eps 1e-5
    assert torch.equal(O.gauss_inverse_transform(x), x * (1.0 + 1e-5))


def test_full_model_applies_normalizer_statistics():
    """galerkin_transformer_2d with mean != 0, std != 1: interior = affine map of the
    default-statistics output, boundary still zero (network/model.py:165-171)."""
    p, i, out, meta = load_golden("galerkin_transformer_2d")
    cfg = dict(meta)
    cfg["resolution_size"] = meta["resolution_size"].tolist()
    base = O.galerkin_transformer_2d(p, cfg, i["x"], i["position"], i["grid"])
    cfg2 = dict(cfg, normalizer_mean=0.7, normalizer_std=2.5, normalizer_eps=1e-5)
    got = O.galerkin_transformer_2d(p, cfg2, i["x"], i["position"], i["grid"])
    inner = (slice(None), slice(1, -1), slice(1, -1))
    want = base[inner] / (1.0 + 1e-5) * (2.5 + 1e-5) + 0.7
    torch.testing.assert_close(got[inner], want, rtol=1e-5, atol=1e-6)
    assert (got[:, 0] == 0).all() and (got[:, -1] == 0).all() and (got[:, :, 0] == 0).all()
