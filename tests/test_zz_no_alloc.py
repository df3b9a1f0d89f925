"""The allocation-free fused attention entry point (partial tiles in the library's own device
array) against the entry point with a caller workspace: same kernels, same plan, so the results
must be bit-identical; and against the fp64 oracle.  Two calls in a row, the second smaller, so
that stale contents of the shared array would show."""
import ctypes

import pytest
import torch

from conftest import max_rel
from oracle import spgt_oracle as O
from spgt_amd import _lib

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32)


def _inputs(B, S, H, seed, dev):
    q, k, v = rnd(B, S, H * 32, seed=seed), rnd(B, S, H * 32, seed=seed + 1) * 1.3 + 0.2, rnd(B, S, H * 32, seed=seed + 2)
    pos = torch.rand(B, S, 2, generator=torch.Generator().manual_seed(seed + 3))
    aff = [1 + 0.3 * rnd(H, 32, seed=seed + 4), 0.2 * rnd(H, 32, seed=seed + 5), 1 + 0.3 * rnd(H, 32, seed=seed + 6),
           0.2 * rnd(H, 32, seed=seed + 7)]
    return [t.to(dev) for t in (q, k, v, pos)], [t.to(dev) for t in aff]


def _call(lib, static, q, k, v, pos, aff, eps, B, S, H, dp):
    D = dp + 32
    out = torch.full((B, S, H * D), float("nan"), device=q.device)
    ktv = torch.full((B, H, D, D), float("nan"), device=q.device)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    pos_ptr = p(pos) if dp else None
    if static:
        rc = lib.spgt_galerkin_attention_fused_forward_static(
            p(q), p(k), p(v), H * 32, pos_ptr, p(aff[0]), p(aff[1]), p(aff[2]), p(aff[3]), eps, p(out), p(ktv),
            B, S, H, dp, stream)
    else:
        need = lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dp)
        ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        rc = lib.spgt_galerkin_attention_fused_forward(
            p(q), p(k), p(v), H * 32, pos_ptr, p(aff[0]), p(aff[1]), p(aff[2]), p(aff[3]), eps, p(out), p(ktv),
            p(ws), need, B, S, H, dp, stream)
    _lib.check(rc)
    torch.cuda.synchronize()
    return out, ktv


# two calls in a row, the second smaller than the first; the second pair starts on the long-sequence plan of the
# K/V pass (1024-thread workgroups) and falls back to the short one
@pytest.mark.parametrize("calls", [[(3, 6007), (2, 1531)], [(2, 150001), (1, 9001)]])
@pytest.mark.parametrize("dp", [0, 2])
def test_static_scratch_entry_point_matches_workspace_entry_point(gpu, dp, calls):
    lib = _lib.load()
    H, eps = 4, 1e-6
    assert lib.spgt_galerkin_attention_fused_static_max_bytes() == 16 << 20
    for call, (B, S) in enumerate(calls):
        print(f"static scratch: call {call} B={B} S={S} dp={dp}", flush=True)
        (q, k, v, pos), aff = _inputs(B, S, H, 100 + 10 * call, gpu)
        assert lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dp) <= 16 << 20
        got, got_ktv = _call(lib, True, q, k, v, pos, aff, eps, B, S, H, dp)
        want, want_ktv = _call(lib, False, q, k, v, pos, aff, eps, B, S, H, dp)
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        assert torch.equal(got_ktv.view(torch.int32), want_ktv.view(torch.int32))
        c = lambda t: t.cpu().double()
        posd = c(pos) if dp else torch.zeros(B, S, 0, dtype=torch.float64)
        ref = O.attention_core_token_major(c(q), c(k), c(v), posd, *(c(a) for a in aff), eps, H)
        assert max_rel(c(got), ref) < 1e-4


def test_static_scratch_entry_point_rejects_oversized_shapes(gpu):
    lib = _lib.load()
    B, S, H = 1200, 64, 4  # one 4 KiB tile per (batch, head): 4800 tiles, more than 16 MiB
    assert lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, 0) > 16 << 20
    t = torch.zeros(16, device=gpu)
    p = ctypes.c_void_p(t.data_ptr())
    rc = lib.spgt_galerkin_attention_fused_forward_static(p, p, p, 128, None, p, p, p, p, 1e-6, p, p, B, S, H, 0, None)
    assert rc == -2 and "static" in _lib.last_error()


def test_static_scratch_entry_point_leaves_device_memory_alone(gpu):
    """After a GPU's first call (one-time set-up: symbol lookup, kernel attribute) the entry point must neither
    take nor give back device memory: free memory as the driver reports it, and torch's own allocator statistics,
    are the same before and after calls on both plans of the K/V pass."""
    lib = _lib.load()
    H, eps = 4, 1e-6
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for dp, (B, S) in ((0, (2, 150001)), (2, (2, 150001)), (2, (3, 6007))):
        D = dp + 32
        (q, k, v, pos), aff = _inputs(B, S, H, 300, gpu)
        out = torch.empty(B, S, H * D, device=gpu)
        ktv = torch.empty(B, H, D, D, device=gpu)
        args = (p(q), p(k), p(v), H * 32, p(pos) if dp else None, p(aff[0]), p(aff[1]), p(aff[2]), p(aff[3]), eps,
                p(out), p(ktv), B, S, H, dp, stream)
        _lib.check(lib.spgt_galerkin_attention_fused_forward_static(*args))  # first call of this kind
        torch.cuda.synchronize()
        free0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        for _ in range(3):
            _lib.check(lib.spgt_galerkin_attention_fused_forward_static(*args))
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_reserved() == reserved0
