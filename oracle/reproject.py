"""Oracle for the q-only / kv-only projections (test infrastructure only).

Reference: additional_designs/model_executor/layers/aptserve_linear.py:102-132.
``weight`` is the fused QKV weight ``[3*Hd, Hd]`` (row-major ``[out, in]``) and
``bias`` is ``[3*Hd]`` or ``None``.  ``slice_ = weight.shape[0] // 3``
(``:116,124``).

* ``q_only``:  ``F.linear(x, weight[:slice_], bias[:slice_])``  (``:115-122``)
* ``kv_only``: ``F.linear(x, weight[slice_:], bias[slice_:])``  (``:123-130``);
  the caller splits the result with ``chunk(2, dim=-1)`` into K and V
  (additional_designs/model_executor/models/aptserve_opt.py:123-124).

The reference runs this in fp16 on the GPU, i.e. fp16 operands, fp32
accumulation inside the BLAS library, fp16 result.  The oracle computes the
exact fp32 product of the fp16-rounded operands and rounds once to the output
dtype; a kernel is compared within 1e-3 relative (before the output rounding)
or 2e-2 absolute (after it).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def _linear_fp32(x, w, b):
    out = F.linear(x.to(torch.float32), w.to(torch.float32),
                   None if b is None else b.to(torch.float32))
    return out


def q_only(x, weight, bias=None, out_dtype=None, keep_fp32: bool = False):
    s = weight.shape[0] // 3
    out = _linear_fp32(x, weight[:s], None if bias is None else bias[:s])
    return out if keep_fp32 else out.to(out_dtype or x.dtype)


def kv_only(x, weight, bias=None, out_dtype=None, keep_fp32: bool = False):
    s = weight.shape[0] // 3
    out = _linear_fp32(x, weight[s:], None if bias is None else bias[s:])
    return out if keep_fp32 else out.to(out_dtype or x.dtype)


def kv_reproject(x, w_kv, b_kv=None, out_dtype=None, keep_fp32: bool = False):
    """``x [T,Hd] @ w_kv[2Hd,Hd]^T + b_kv`` -> ``(k [T,Hd], v [T,Hd])``."""
    out = _linear_fp32(x, w_kv, b_kv)
    if not keep_fp32:
        out = out.to(out_dtype or x.dtype)
    k, v = out.chunk(2, dim=-1)
    return k, v
