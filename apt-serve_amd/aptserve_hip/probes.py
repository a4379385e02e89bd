"""ctypes binding of libaptserve_probes.so: the benchmark's measurement kernels (plain copy / read / fill
streams, bare matrix-core instruction streams).  Kept apart from the operators: nothing of the hybrid-cache
path imports this module; ``bench.py`` and the tests of the probes themselves do.  Prototypes come from
``include/aptserve_probes.h``."""

from __future__ import annotations

import ctypes

import torch

from . import _lib

HEADER = _lib.HEADER.parent / "aptserve_probes.h"
LIB_PATH = _lib.PKG_DIR / "libaptserve_probes.so"

_probes = None


def load() -> ctypes.CDLL:
    global _probes
    if _probes is None:
        _lib.load()  # the product library first: both must bind to the HIP runtime torch loaded
        _probes, _ = _lib.bind(LIB_PATH, HEADER)
    return _probes


def copy_bytes(dst: torch.Tensor, src: torch.Tensor) -> None:
    """Plain device copy (the kernel of known traffic that hardware counters are scaled against)."""
    if not (dst.is_cuda and src.is_cuda and dst.device == src.device):
        raise ValueError("both tensors must be on one GPU")
    if not (dst.is_contiguous() and src.is_contiguous()):
        raise ValueError("tensors must be contiguous")
    nbytes = src.numel() * src.element_size()
    if nbytes != dst.numel() * dst.element_size():
        raise ValueError("sizes differ")
    with torch.cuda.device(src.device):
        st = load().aps_copy_bytes(dst.data_ptr(), src.data_ptr(), nbytes,
                                   torch.cuda.current_stream(src.device).cuda_stream)
    _lib.check(st, "copy_bytes")
