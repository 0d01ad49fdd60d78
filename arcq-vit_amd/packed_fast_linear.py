"""``ARCQPackedLinearFast``: same storage as ``ARCQPackedLinear``; forward rebuilds the dense
weight, then runs a plain fp32 ``F.linear`` on the UNQUANTIZED activation
(FQ/arcq_packed_fast_linear.py:14-45 -- that variant never quantizes x).

The weight rebuild is the HIP stage-2 kernel (fp32 arithmetic, one rounding to fp16); the
reference does the same formula in fp16 arithmetic (:48-93), which can differ by an fp16 ulp.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import ops
from .packed_linear import ARCQPackedLinear


class ARCQPackedLinearFast(ARCQPackedLinear):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        original_shape = x.shape
        if original_shape[-1] != self.in_features:
            raise ValueError(f"expected last dim {self.in_features}, got {original_shape[-1]}")
        device = self.packed_weight_codes.device
        x_fp32 = x.reshape(-1, self.in_features).to(device=device, dtype=torch.float32)
        w_fp16 = ops.unpack_weight_hip(self.packed_weight_codes, self.weight_codebook, self.weight_center,
                                       self.weight_scale, self.weight_code_sum, self.bits, self.group_size)
        bias = self.bias if self.bias.numel() > 0 else None
        y = F.linear(x_fp32, w_fp16.to(dtype=torch.float32), bias)
        return y.reshape(*original_shape[:-1], self.out_features)
