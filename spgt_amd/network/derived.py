"""Derived operand layouts of module parameters.

Several kernels take a parameter in another layout than nn.Module stores it in: nn.Linear weights
transposed to [in, out], the three projection weights packed side by side, a 3x3 convolution's weight as
nine [Cin, Cout] taps.  Such a copy must never go stale, and a parameter can change without any trace on
the host (`w.data.mul_(2)`, an optimizer step through `.data`, `load_state_dict` all leave `_version`
alone).  So the copies are not cached by key: every inference forward starts with ONE launch that
rewrites all derived tensors of the module tree from the parameters as they are now (a few hundred KB
read out of the caches), and a derived tensor requested outside such a forward is rewritten on the spot.
The derived tensors keep their addresses for as long as the parameters keep theirs, so a captured HIP
graph, which replays that launch too, follows in-place parameter updates.
"""
import functools
import threading
from typing import Callable, List, Sequence, Tuple

import torch
from torch import Tensor, nn

from .. import _lib

# (source, source offset, sizes[3], source strides[3], destination offset, destination strides[3]), in elements
Copy = Tuple[Tensor, int, Sequence[int], Sequence[int], int, Sequence[int]]

_tls = threading.local()
_generation = [0]


def _signature(shape, copies: List[Copy]) -> tuple:
    """What a derived tensor was built from: the storage address, dtype, device and strided view of every
    source as the spec names them now.  A parameter object that was replaced (load_state_dict(assign=True),
    `lin.weight = nn.Parameter(...)`, parametrizations) or whose strides changed gives another signature."""
    return (tuple(shape),) + tuple(
        (src.data_ptr(), src.dtype, src.device, soff, tuple(size), tuple(sstr), doff, tuple(dstr))
        for src, soff, size, sstr, doff, dstr in copies)


class _Entry:
    __slots__ = ("dst", "spec", "sig", "descs", "stamp")

    def __init__(self, spec, shape, copies: List[Copy], sig) -> None:
        device = copies[0][0].device
        self.dst = torch.empty(shape, dtype=torch.float32, device=device)
        self.spec = spec
        self.sig = sig
        self.stamp = -1
        self.descs = []
        for src, soff, size, sstr, doff, dstr in copies:
            if src.dtype != torch.float32 or src.device != device:
                raise TypeError("derived weights need float32 sources on one device")
            d = _lib.CopyDesc()
            d.src = src.data_ptr() + 4 * soff
            d.dst = self.dst.data_ptr() + 4 * doff
            d.size[:] = list(size)
            d.src_stride[:] = list(sstr)
            d.dst_stride[:] = list(dstr)
            self.descs.append(d)

    def valid(self) -> bool:
        """True when the spec, consulted now, still names the sources this entry copies from.  The spec
        re-resolves the parameters through their modules, so a replaced parameter is seen."""
        return _signature(*self.spec()) == self.sig


def _launch(descs: Sequence, device) -> None:
    if not descs:
        return
    arr = (_lib.CopyDesc * len(descs))(*descs)
    with _lib.device_guard(device):
        _lib.check(_lib.load().spgt_strided_copy_batch(
            arr, len(descs), torch.cuda.current_stream(device).cuda_stream))


def derived(module: nn.Module, name: str, spec: Callable[[], Tuple[Sequence[int], List[Copy]]]) -> Tensor:
    """The derived tensor `name` of `module`, up to date with its sources.  `spec()` gives its shape and the
    strided copies that fill it, and must look the parameters up through their modules every time it is called
    (it is kept and consulted again by every later refresh, to see parameters that were replaced)."""
    table = module.__dict__.setdefault("_spgt_derived", {})
    ent = table.get(name)
    active = getattr(_tls, "active", False)
    if ent is not None and active and ent.stamp == getattr(_tls, "forward_id", -2):
        return ent.dst  # checked and rewritten by the refresh that opened this forward
    shape, copies = spec()
    sig = _signature(shape, copies)
    if ent is None or ent.sig != sig:
        ent = _Entry(spec, shape, copies, sig)
        table[name] = ent
        _generation[0] += 1
        _launch(ent.descs, ent.dst.device)
    elif not active:
        _launch(ent.descs, ent.dst.device)  # no forward-level refresh is covering this request
    return ent.dst


def refresh(root: nn.Module) -> None:
    """Rewrites every derived tensor under `root` from its sources, in one launch per 64 copies.  Entries
    whose sources are no longer the ones they were built from are dropped; their next request rebuilds them."""
    cache = root.__dict__.get("_spgt_refresh")
    if cache is None or cache[0] != _generation[0]:
        entries = [e for m in root.modules() for e in m.__dict__.get("_spgt_derived", {}).values()]
        cache = (_generation[0], entries, [d for e in entries for d in e.descs])
        root.__dict__["_spgt_refresh"] = cache
    _, entries, descs = cache
    if not entries:
        return
    if not all(e.valid() for e in entries):
        # a source moved (new parameter object, new storage, other strides, another device)
        for m in root.modules():
            table = m.__dict__.get("_spgt_derived")
            if table:
                for k in [k for k, e in table.items() if not e.valid()]:
                    del table[k]
        _generation[0] += 1
        return refresh(root)
    _launch(descs, entries[0].dst.device)
    stamp = getattr(_tls, "forward_id", -2)
    for e in entries:
        e.stamp = stamp


_forward_counter = [0]


def refreshes_derived(forward):
    """Decorator for a module's forward: the outermost decorated forward of a call tree refreshes the derived
    tensors of its whole subtree first; nested ones rely on it."""

    @functools.wraps(forward)
    def wrapper(self, *args, **kwargs):
        if getattr(_tls, "active", False):
            return forward(self, *args, **kwargs)
        _tls.active = True
        _forward_counter[0] += 1
        _tls.forward_id = _forward_counter[0]
        try:
            refresh(self)
            with _lib.seed_scope():
                return forward(self, *args, **kwargs)
        finally:
            _tls.active = False
            _tls.forward_id = -2

    return wrapper


def transposed_2d(w: Tensor, rows: slice = None) -> Tuple[Sequence[int], List[Copy]]:
    """Spec of w[:, cols]^T for a 2-D parameter w [out, in]: dst [n_cols, out] contiguous."""
    out_f, in_f = w.shape
    c0, c1 = (0, in_f) if rows is None else (rows.start, rows.stop)
    n = c1 - c0
    return (n, out_f), [(w, c0 * w.stride(1), (1, n, out_f), (0, w.stride(1), w.stride(0)), 0, (0, out_f, 1))]
