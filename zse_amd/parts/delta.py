"""A recurrent mixer with a matrix state per head, written by the gated delta rule.

Per value head, D query/key channels and E value channels; the state S [D, E] starts at zero and
is carried as floats in the request's state slot:

    q, k, v = silu(conv(W_q x)), silu(conv(W_k x)), silu(conv(W_v x))        (a short causal convolution per channel)
    q <- q / sqrt(sum q^2 + 1e-6) D^(-1/2),   k <- k / sqrt(sum k^2 + 1e-6)    (per head)
    beta = sigmoid(W_b x),   g = exp(-exp(A) softplus(W_a x + dt))            (per head, float)
    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
    out = W_o ( o / sqrt(mean(o^2) + eps) * gain * silu(W_g x) )              (the mean per head)

Value head h reads query/key head h // (heads / kv_heads).  q, k, v and the gate are one
product; b and a a second, small one whose results stay float.  The convolution's last
``taps - 1`` inputs are part of the request's state, behind S.  One kernel walks the tokens of
every (request, head): eight lanes own a column of S, so steps of single tokens and portions of
prompts run the same arithmetic in the same order.
"""
from __future__ import annotations

from typing import List

from ..config.plan import ShortConvSpec
from ..runtime.device import F32, Tensor
from .base import ROLE_GAIN, Part, StateNeed, TensorReq, build_part, register_part
from .ops import linear


class DeltaRule(Part):
    graph_safe = True      # rows, requests and slots are read by the kernels from device memory

    def __init__(self, spec):
        s = self.spec = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"heads ({s.num_heads}) must be a multiple of kv_heads ({s.num_kv_heads})")
        if s.key_dim > 256 or s.value_dim > 1024:
            raise ValueError(f"up to 256 key and 1024 value channels a head, got {s.key_dim} and {s.value_dim}")
        n = s.names
        self.qk = s.num_kv_heads * s.key_dim
        self.vv = s.num_heads * s.value_dim
        self.conv = build_part("filter", ShortConvSpec(
            size=2 * self.qk + self.vv, taps=s.conv_taps, weight=(n["q_conv"], n["k_conv"], n["v_conv"]),
            residual=False, activation="silu", channel_counts=(self.qk, self.qk, self.vv)))
        self.w_in = self.w_ba = self.w_o = None
        self.A_log = self.dt_bias = self.gain = None

    def children(self):
        return [self.conv]

    def tensor_reqs(self) -> List[TensorReq]:
        s, n = self.spec, self.spec.names
        H, W = s.num_heads, s.hidden_size
        return [TensorReq(n["q"], (self.qk, W)), TensorReq(n["k"], (self.qk, W)), TensorReq(n["v"], (self.vv, W)),
                TensorReq(n["gate"], (self.vv, W)), TensorReq(n["o"], (W, self.vv)),
                TensorReq(n["b"], (H, W)), TensorReq(n["a"], (H, W)),
                TensorReq(n["A_log"], (H,), ROLE_GAIN), TensorReq(n["dt_bias"], (H,), ROLE_GAIN),
                TensorReq(n["norm"], (s.value_dim,), ROLE_GAIN)]

    def load(self, weights, rt, dtype):
        s, n = self.spec, self.spec.names
        strip = getattr(weights, "wants_strip", None)
        wide = bool(strip and strip(s.hidden_size))
        self.w_in = weights.matrix([n["q"], n["k"], n["v"], n["gate"]], strip=wide)
        self.w_ba = weights.matrix([n["b"], n["a"]], strip=wide)
        self.w_o = weights.matrix([n["o"]], strip=bool(strip and strip(self.vv)))
        self.A_log, self.dt_bias = weights.vector(n["A_log"]), weights.vector(n["dt_bias"])
        self.gain = weights.vector(n["norm"])

    def state_words(self) -> int:
        s = self.spec
        return s.num_heads * s.key_dim * s.value_dim

    def cache_need(self):
        # S of every head, then the convolution's rows
        return StateNeed(self.state_words() * 4 + self.conv.state_bytes())

    def flops_per_token(self) -> float:
        s = self.spec
        return super().flops_per_token() + 6.0 * s.num_heads * s.key_dim * s.value_dim    # S^T k, k u^T, S^T q

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        H, G, D, E = s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim
        ld = 2 * self.qk + 2 * self.vv
        qkvz = linear(ctx, x, self.w_in, ctx.alloc((T, ld)))
        ba = linear(ctx, x, self.w_ba, ctx.alloc((T, 2 * H), F32))
        qkv = self.conv.forward(ctx, qkvz, cache.state_offset + self.state_words() * 4, ld=ld)
        out = ctx.alloc((T, self.vv))
        z_ptr = qkvz.ptr + (2 * self.qk + self.vv) * (4 if ctx.dtype == F32 else 2)
        # read-outs before their norm, for steps in which a head's value channels spread over several blocks
        raw = ctx.alloc((T, self.vv), F32) if (E > 64 or ctx.max_q_len > 16) else None
        k.zk_delta_rule(qkv.ptr, 2 * self.qk + self.vv, self.qk, 2 * self.qk, z_ptr, ld, ba.ptr, self.A_log.ptr,
                        self.dt_bias.ptr, self.gain.ptr, ctx.state.ptr, ctx.state.shape[1], cache.state_offset // 4,
                        ctx.q_start, ctx.slot_of_req, ctx.positions, out.ptr, raw.ptr if raw is not None else None, T,
                        ctx.R, int(ctx.max_q_len), H, G, D, E, float(s.eps), ctx.stream)
        return linear(ctx, out, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "delta_rule", DeltaRule)
