"""A layer over several residual streams (hyper-connections).

The float residual holds S rows per token.  Sublayer q (1: the mixer, 2: the feed-forward)
reads u = sum_s in_q[s] x_s, computes y = sublayer(norm_q(u)) and writes every stream from the
old ones, x_r <- sum_s mix_q[s, r] x_s + out_q[r] y.  One kernel does a sublayer's write and
the next sublayer's read and norm, also across the boundary to the next layer.  Without
streams (S = 1, unit weights) this is the pre-norm residual layer with layer norms.  A short
convolution over time may sit between the first norm and the mixer; what it keeps per request
is part of the layer's state.
"""
from __future__ import annotations

from typing import List

import numpy as np

from ..runtime.device import Tensor
from .base import ROLE_GAIN, Part, TensorReq, build_part, register_part
from .norm import LayerNorm


class StreamsBlock(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec
        self.S = int(spec.streams or 1)
        if not (1 <= self.S <= 8):
            raise ValueError(f"1 to 8 residual streams, got {spec.streams}")
        self.norms = {"pre_mixer": build_part("norm", spec.norms["pre_mixer"])}
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        if self.ffn is not None:
            self.norms["pre_ffn"] = build_part("norm", spec.norms["pre_ffn"])
        for n in self.norms.values():
            if not isinstance(n, LayerNorm):
                raise ValueError("a streams block reads through layer norms")
        self.conv = build_part("filter", spec.conv) if spec.conv is not None else None
        self.size = self.norms["pre_mixer"].spec.size
        self.w = {}

    def children(self):
        out = list(self.norms.values()) + [self.mixer]
        if self.ffn is not None:
            out.append(self.ffn)
        if self.conv is not None:
            out.append(self.conv)
        return out

    def _sublayers(self):
        return (1, 2) if self.ffn is not None else (1,)

    def tensor_reqs(self) -> List[TensorReq]:
        if self.spec.streams is None:
            return []
        S, n = self.S, self.spec.names
        out = []
        for q in self._sublayers():
            out += [TensorReq(n[f"in{q}"], (S,), ROLE_GAIN), TensorReq(n[f"out{q}"], (S,), ROLE_GAIN),
                    TensorReq(n[f"mix{q}"], (S, S), ROLE_GAIN)]
        return out

    def load(self, weights, rt, dtype):
        if self.spec.streams is None:
            one = rt.upload(np.ones((1,), np.float32))
            self.w = {f"{r}{q}": one for r in ("in", "out", "mix") for q in (1, 2)}
        else:
            self.w = {f"{r}{q}": weights.vector(self.spec.names[f"{r}{q}"])
                      for r in ("in", "out", "mix") for q in self._sublayers()}

    def state_needs(self):
        return [("conv", self.conv.state_bytes())] if self.conv is not None and self.conv.state_bytes() else []

    def entry_norm(self):
        """What the layer before needs to read the streams for this one's mixer in the kernel
        that ends its own work: this block (its first read's weights and norm)."""
        return self

    def _step(self, ctx, h: Tensor, y, q_write, reader, q_read, out: Tensor = None):
        """Write sublayer ``q_write``'s result ``y`` into the streams (None: nothing to write) and
        read them for sublayer ``q_read`` of ``reader`` (None: no read).  Returns the normed read."""
        T, W = h.shape[0], self.size
        norm = reader.norms["pre_mixer" if q_read == 1 else "pre_ffn"] if reader is not None else None
        if norm is not None:
            out = ctx.alloc((T, W)) if out is None else Tensor(out.ptr, (T, W), ctx.dtype, out.owner)
        parts = y.shape[0] if (y is not None and y.layout == "parts") else 0
        ctx.k.zk_streams_step(
            h.ptr, self.S, y.ptr if y is not None else None, parts,
            self.w[f"mix{q_write}"].ptr if y is not None else None, self.w[f"out{q_write}"].ptr if y is not None else None,
            reader.w[f"in{q_read}"].ptr if reader is not None else None,
            norm.weight.ptr if norm is not None else None,
            norm.bias.ptr if (norm is not None and norm.bias is not None) else None,
            norm.spec.eps if norm is not None else 0.0, None, out.ptr if norm is not None else None, T, T, W, ctx.stream)
        return out if norm is not None else None

    def forward(self, ctx, h: Tensor, cache, x_in: Tensor = None, next_norm=None, x_out: Tensor = None):
        """Update the streams ``h`` [T, S * W] in place.  ``x_in``: this block's first read,
        if the caller has it.  ``next_norm``: the block that runs next (its ``entry_norm()``);
        its first read is returned, made by the kernel that writes this block's last result."""
        x = x_in if x_in is not None else self._step(ctx, h, None, 0, self, 1)
        if self.conv is not None:
            x = self.conv.forward(ctx, x, cache.extra["conv"][0] if "conv" in cache.extra else 0)
        ctx.sums_welcome = self.mixer          # the kernel that writes the streams adds partial sums up itself
        y, q = self.mixer.forward(ctx, x, cache), 1
        if self.ffn is not None:
            x = self._step(ctx, h, y, 1, self, 2)
            ctx.sums_welcome = self.ffn
            y, q = self.ffn.forward(ctx, x), 2
        ctx.sums_welcome = None
        nxt = next_norm if (isinstance(next_norm, StreamsBlock) and next_norm.S == self.S
                            and next_norm.size == self.size) else None
        return self._step(ctx, h, y, q, nxt, 1, out=x_out)


register_part("block", "streams", StreamsBlock)
