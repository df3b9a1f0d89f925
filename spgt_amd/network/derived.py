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


class _Entry:
    __slots__ = ("dst", "srcs", "ptrs", "descs")

    def __init__(self, shape, copies: List[Copy]) -> None:
        device = copies[0][0].device
        self.dst = torch.empty(shape, dtype=torch.float32, device=device)
        self.srcs = [c[0] for c in copies]
        self.ptrs = tuple(s.data_ptr() for s in self.srcs)
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
        for s, p in zip(self.srcs, self.ptrs):
            if s.data_ptr() != p:
                return False
        return True


def _launch(descs: Sequence, device) -> None:
    if not descs:
        return
    arr = (_lib.CopyDesc * len(descs))(*descs)
    with torch.cuda.device(device):
        _lib.check(_lib.load().spgt_strided_copy_batch(
            arr, len(descs), torch.cuda.current_stream(device).cuda_stream))


def derived(module: nn.Module, name: str, spec: Callable[[], Tuple[Sequence[int], List[Copy]]]) -> Tensor:
    """The derived tensor `name` of `module`, up to date with its sources.  `spec()` gives its shape and the
    strided copies that fill it; it is consulted when the tensor does not exist yet or a source has moved."""
    table = module.__dict__.setdefault("_spgt_derived", {})
    ent = table.get(name)
    if ent is None or not ent.valid():
        shape, copies = spec()
        ent = _Entry(shape, copies)
        table[name] = ent
        _generation[0] += 1
        _launch(ent.descs, ent.dst.device)
    elif not getattr(_tls, "active", False):
        _launch(ent.descs, ent.dst.device)  # no forward-level refresh is covering this request
    return ent.dst


def refresh(root: nn.Module) -> None:
    """Rewrites every derived tensor under `root` from its sources, in one launch per 64 copies."""
    cache = root.__dict__.get("_spgt_refresh")
    if cache is None or cache[0] != _generation[0]:
        entries = [e for m in root.modules() for e in m.__dict__.get("_spgt_derived", {}).values()]
        cache = (_generation[0], entries, [d for e in entries for d in e.descs])
        root.__dict__["_spgt_refresh"] = cache
    _, entries, descs = cache
    if not entries:
        return
    if not all(e.valid() for e in entries):
        # a source moved (new storage, another device): drop those tensors, their next request rebuilds them
        for m in root.modules():
            table = m.__dict__.get("_spgt_derived")
            if table:
                for k in [k for k, e in table.items() if not e.valid()]:
                    del table[k]
        _generation[0] += 1
        return refresh(root)
    _launch(descs, entries[0].dst.device)


def refreshes_derived(forward):
    """Decorator for a module's forward: the outermost decorated forward of a call tree refreshes the derived
    tensors of its whole subtree first; nested ones rely on it."""

    @functools.wraps(forward)
    def wrapper(self, *args, **kwargs):
        if getattr(_tls, "active", False):
            return forward(self, *args, **kwargs)
        _tls.active = True
        try:
            refresh(self)
            return forward(self, *args, **kwargs)
        finally:
            _tls.active = False

    return wrapper


def transposed_2d(w: Tensor, rows: slice = None) -> Tuple[Sequence[int], List[Copy]]:
    """Spec of w[:, cols]^T for a 2-D parameter w [out, in]: dst [n_cols, out] contiguous."""
    out_f, in_f = w.shape
    c0, c1 = (0, in_f) if rows is None else (rows.start, rows.stop)
    n = c1 - c0
    return (n, out_f), [(w, c0 * w.stride(1), (1, n, out_f), (0, w.stride(1), w.stride(0)), 0, (0, out_f, 1))]
