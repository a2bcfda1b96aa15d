"""A recurrent mixer with a matrix memory per head (the mLSTM of xLSTM).

Per head, D query/key channels and E value channels; the state (S [D, E], n [D], m) starts
at zero and is carried as floats in the request's state slot:

    i_t = cap tanh((W_i x_t + b_i) / cap)          f_t = logsigmoid(cap tanh((W_f x_t + b_f) / cap))
    m_t = max(f_t + m_(t-1), i_t)
    S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T      (n_t likewise with k_t)
    o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),    q_t = W_q x_t D^(-1/2)
    out = W_o ( o_t / sqrt(mean(o_t^2) + eps) * g * sigmoid(W_z x_t) )      (the mean per head)

q, k, v and z are one product; the two gates are a second, small one whose results stay float.
Steps of single tokens run the recurrence as written, one block per (request, head); steps with
portions of prompts run it over chunks of up to 64 tokens, where it becomes four small matrix
products per chunk, with a head's value channels spread over several blocks; portions of several
chunks run all their chunks at once around a short scan that carries the state from chunk to chunk.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import BF16, F32, Tensor
from .base import ROLE_GAIN, Part, StateNeed, TensorReq, register_part
from .ops import linear


class MatrixMemory(Part):
    graph_safe = True      # rows, requests and slots are read by the kernel from device memory
    SCAN_FROM = 64         # portions longer than this (more than one chunk) run their chunks side by side

    def __init__(self, spec):
        s = self.spec = spec
        if s.value_dim > 256:
            raise ValueError(f"up to 256 value channels a head, got {s.value_dim}")
        if not s.gate_cap > 0:
            raise ValueError(f"the gates' cap must be positive, got {s.gate_cap}")
        self.w_qkvz = self.w_gates = self.w_o = None
        self.bias_i = self.bias_f = self.gain = None

    def tensor_reqs(self) -> List[TensorReq]:
        s, n = self.spec, self.spec.names
        H, D, E, W = s.num_heads, s.key_dim, s.value_dim, s.hidden_size
        return [TensorReq(n["q"], (H * D, W)), TensorReq(n["k"], (H * D, W)), TensorReq(n["v"], (H * E, W)),
                TensorReq(n["gate"], (H * E, W)), TensorReq(n["o"], (W, H * E)),
                TensorReq(n["norm"], (H * E,), ROLE_GAIN),
                TensorReq(n["i"], (H, W)), TensorReq(n["i_bias"], (H,), ROLE_GAIN),
                TensorReq(n["f"], (H, W)), TensorReq(n["f_bias"], (H,), ROLE_GAIN)]

    def load(self, weights, rt, dtype):
        s, n = self.spec, self.spec.names
        strip = getattr(weights, "wants_strip", None)
        wide = bool(strip and strip(s.hidden_size))
        self.w_qkvz = weights.matrix([n["q"], n["k"], n["v"], n["gate"]], strip=wide)
        self.w_gates = weights.matrix([n["i"], n["f"]], strip=wide)
        self.w_o = weights.matrix([n["o"]], strip=bool(strip and strip(s.num_heads * s.value_dim)))
        self.bias_i, self.bias_f = weights.vector(n["i_bias"]), weights.vector(n["f_bias"])
        self.gain = weights.vector(n["norm"])

    def cache_need(self):
        s = self.spec
        return StateNeed(s.num_heads * (s.key_dim * s.value_dim + s.key_dim + 1) * 4)

    def flops_per_token(self) -> float:
        s = self.spec
        return super().flops_per_token() + 4.0 * s.num_heads * s.key_dim * s.value_dim    # the state's update and read-out

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        H, D, E = s.num_heads, s.key_dim, s.value_dim
        ld = 2 * H * (D + E)
        qkvz = linear(ctx, x, self.w_qkvz, ctx.alloc((T, ld)))
        gates = linear(ctx, x, self.w_gates, ctx.alloc((T, 2 * H), F32))
        out = ctx.alloc((T, H * E))
        words, at = ctx.state.shape[1], cache.state_offset // 4
        if ctx.max_q_len > 1 and ctx.dtype == BF16 and D <= 256:
            # a step with portions of prompts: chunks of tokens as small matrix products, then the
            # heads' norm and gate.  (In 32-bit every step runs token by token, so that a request's
            # values are the same bits however its tokens are cut into steps.)
            o_raw = ctx.alloc((T, H * E), F32)
            if ctx.max_q_len > self.SCAN_FROM:
                # portions of several chunks: every chunk's own part at once, a short scan over the
                # chunks, every chunk's read-out at once
                floats = int(k.zk_mlstm_scan_floats(T, ctx.R, H, D, E, int(ctx.max_q_len)))
                work = ctx.alloc((floats,), F32)
                k.zk_mlstm_scan(qkvz.ptr, ld, gates.ptr, self.bias_i.ptr, self.bias_f.ptr, ctx.state.ptr, words, at,
                                ctx.q_start, ctx.slot_of_req, o_raw.ptr, work.ptr, floats, T, ctx.R, H, D, E,
                                float(s.gate_cap), int(ctx.max_q_len), ctx.stream)
                nm_ptr = None
            else:
                nm = ctx.alloc((ctx.R, H * (D + 1)), F32)
                k.zk_mlstm_chunked(qkvz.ptr, ld, gates.ptr, self.bias_i.ptr, self.bias_f.ptr, ctx.state.ptr, words, at,
                                   ctx.q_start, ctx.slot_of_req, o_raw.ptr, nm.ptr, ctx.R, H, D, E, float(s.gate_cap),
                                   int(ctx.max_q_len), ctx.stream)
                nm_ptr = nm.ptr
            k.zk_mlstm_finish(o_raw.ptr, qkvz.ptr, ld, self.gain.ptr, nm_ptr, ctx.state.ptr, words, at, ctx.req_of_token,
                              ctx.q_start, ctx.slot_of_req, out.ptr, T, H, D, E, float(s.eps), ctx.stream)
        else:
            # steps of single tokens renew the state where it lies; same bits as the staged kernel
            run = k.zk_mlstm_token if ctx.max_q_len == 1 else k.zk_mlstm
            run(qkvz.ptr, ld, gates.ptr, self.bias_i.ptr, self.bias_f.ptr, self.gain.ptr, ctx.state.ptr, words, at,
                ctx.q_start, ctx.slot_of_req, out.ptr, ctx.R, H, D, E, float(s.gate_cap), float(s.eps), ctx.stream)
        return linear(ctx, out, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "mlstm", MatrixMemory)
