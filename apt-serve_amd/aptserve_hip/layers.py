"""Host-side mirrors of the reference's model-side call sites for the hot path.

``QKVLinear`` follows ``ColumnParallelLinear.forward(input_, q_only, kv_only)``
(additional_designs/model_executor/layers/aptserve_linear.py:315-328) with
``UnquantizedLinearMethod.apply`` (``:102-132``): the fused weight is
``[3*Hd, Hd]``; ``q_only`` uses rows ``[:Hd]``, ``kv_only`` rows ``[Hd:]``; the
call returns ``(output, output_bias)`` with ``output_bias = None`` because the
bias is added inside (``skip_bias_add=False``).  Single GPU: no gather.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops


class QKVLinear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2 or weight.size(0) % 3 != 0:
            raise ValueError("fused QKV weight [3*Hd, Hd] expected")
        self.weight = weight
        self.bias = bias

    def __call__(self, input_: torch.Tensor, q_only: bool = False, kv_only: bool = False
                 ) -> Tuple[torch.Tensor, None]:
        if q_only and kv_only:
            raise NotImplementedError          # aptserve_linear.py:131-132
        s = self.weight.shape[0] // 3          # ``slice_`` of :116,124
        if q_only:
            w, b = self.weight[:s], None if self.bias is None else self.bias[:s]
        elif kv_only:
            w, b = self.weight[s:], None if self.bias is None else self.bias[s:]
        else:
            w, b = self.weight, self.bias
        return ops.linear_nt(input_, w, b), None

    forward = __call__
