"""Root-mean-square norm, gain (1 + w) or w; layer norm with gain and bias.

Statistics and the product are float; rsqrt(mean(x^2) + eps) as in the
reference's kernel (orchestrator/kernels.py:1435-1465); the reference multiplies
by plain w and names the (1 + w) form of Gemma 2 in a comment (:1476-1478).
"""
from __future__ import annotations

from typing import List, Optional

from ..runtime.device import F32, Tensor
from .base import ROLE_GAIN, Part, TensorReq, register_part


class RMSNorm(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec
        self.weight: Optional[Tensor] = None

    def tensor_reqs(self) -> List[TensorReq]:
        return [TensorReq(self.spec.weight, (self.spec.size,), ROLE_GAIN)]

    def load(self, weights, rt, dtype):
        self.weight = weights.vector(self.spec.weight)

    def forward(self, ctx, x: Tensor, out_rows=None) -> Tensor:
        """Norm of every row of ``x`` (float stream or activations), or of the rows
        ``out_rows = (device int32 pointer, count)``."""
        s = self.spec
        rows_ptr, n = (out_rows if out_rows is not None else (0, x.shape[0]))
        out = ctx.alloc((n, s.size))
        ctx.k.zk_rmsnorm(x.ptr, 1 if x.dtype == F32 else 0,
                         rows_ptr or None, self.weight.ptr, out.ptr, s.eps,
                         1 if s.unit_offset else 0, n, s.size, ctx.stream)
        return out


class LayerNorm(Part):
    """(x - mean) / sqrt(var + eps) * gain + bias over the float residual; with several residual
    streams a token the norm reads their plain sum."""
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if not (1 <= spec.streams <= 8):
            raise ValueError(f"a layer norm reads 1 to 8 streams, got {spec.streams}")
        self.spec = spec
        self.weight: Optional[Tensor] = None
        self.bias: Optional[Tensor] = None

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        out = [TensorReq(s.weight, (s.size,), ROLE_GAIN)]
        if s.bias:
            out.append(TensorReq(s.bias, (s.size,), ROLE_GAIN))
        return out

    def load(self, weights, rt, dtype):
        self.weight = weights.vector(self.spec.weight)
        self.bias = weights.vector(self.spec.bias) if self.spec.bias else None

    def forward(self, ctx, x: Tensor, out_rows=None) -> Tensor:
        s = self.spec
        if x.dtype != F32 or x.shape[1] != s.streams * s.size:
            raise ValueError(f"layer norm over {s.streams} float streams of {s.size}: got {x.dtype} {x.shape}")
        rows_ptr, n = (out_rows if out_rows is not None else (0, x.shape[0]))
        out = ctx.alloc((n, s.size))
        ctx.k.zk_streams_step(x.ptr, s.streams, None, 0, None, None, None, self.weight.ptr,
                              self.bias.ptr if self.bias is not None else None, s.eps, rows_ptr or None, out.ptr, n,
                              x.shape[0], s.size, ctx.stream)
        return out


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
