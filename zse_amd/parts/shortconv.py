"""A short causal convolution over time on each channel, added to its input:
out_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j), rows before a sequence's start being zero.
The ``taps - 1`` rows before a request's next token are its state (float, in its state slot,
which starts as zeros): a step reads them for its first tokens and renews them afterwards.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import Tensor
from .base import ROLE_GAIN, Part, TensorReq, register_part


class ShortConv(Part):
    graph_safe = True      # rows, requests and slots are read by the kernels from device memory

    def __init__(self, spec):
        if spec.taps < 1:
            raise ValueError(f"a convolution has at least one tap, got {spec.taps}")
        self.spec = spec
        self.weight = None

    def tensor_reqs(self) -> List[TensorReq]:
        return [TensorReq(self.spec.weight, (self.spec.size, self.spec.taps), ROLE_GAIN)]

    def load(self, weights, rt, dtype):
        self.weight = weights.vector(self.spec.weight)

    def state_bytes(self) -> int:
        return (self.spec.taps - 1) * self.spec.size * 4

    def flops_per_token(self) -> float:
        return 2.0 * self.spec.size * self.spec.taps

    def forward(self, ctx, x: Tensor, state_offset: int) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        out = ctx.alloc((T, s.size))
        state = ctx.state.ptr if ctx.state is not None else None
        words = ctx.state.shape[1] if ctx.state is not None else 0
        if ctx.max_q_len == 1 and T == ctx.R:
            # every request brings one token: one launch computes and moves the state on
            k.zk_short_conv_token(x.ptr, self.weight.ptr, state, words, state_offset // 4, ctx.positions,
                                  ctx.req_of_token, ctx.q_start, ctx.slot_of_req, out.ptr, T, s.size, s.taps, ctx.stream)
            return out
        k.zk_short_conv(x.ptr, self.weight.ptr, state, words, state_offset // 4, ctx.positions, ctx.req_of_token,
                        ctx.q_start, ctx.slot_of_req, out.ptr, T, s.size, s.taps, ctx.stream)
        k.zk_short_conv_state(x.ptr, state, words, state_offset // 4, ctx.q_start, ctx.slot_of_req, ctx.R, s.size,
                              s.taps, ctx.stream)
        return out


register_part("filter", "short_conv", ShortConv)
