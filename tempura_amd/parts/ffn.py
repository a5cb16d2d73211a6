"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases
(/root/reference/engine/src/model.rs:1203-1231,1301-1313;
``silu(x) = x / (1 + exp(-x))``, /root/reference/kernels/src/ggml/vec_llama.rs:808-810).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, WeightInfo, register_part


class SwiGLU(FeedForward):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph
    split_norm = True      # takes rows whose norm its first product finishes; prepares the next norm in its last

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.w13 = None
        self.w2 = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        i, w = spec.params["intermediate_size"], spec.weights
        return {
            w["gate"]: WeightInfo((i, hidden_size)),
            w["up"]: WeightInfo((i, hidden_size)),
            w["down"]: WeightInfo((hidden_size, i)),
        }

    def load_weights(self, get):
        w = self.spec.weights
        gate, up = self._to_device(get(w["gate"])), self._to_device(get(w["up"]))
        # One matrix, one product instead of two.  In bfloat16 the rows alternate eight of gate and
        # eight of up, so that the product's epilogue applies silu(g) * u to its float32 sums.
        self.fused = self.dtype == torch.bfloat16 and ops.gated_layout_ok(self.intermediate_size, self.hidden_size)
        if self.fused:
            self.w13 = ops.tile_weight(ops.interleave_gate_up(gate, up))
        else:
            self.w13 = ops.tile_weight(torch.cat([gate, up], dim=0).contiguous())
        self.w2 = ops.tile_weight(self._to_device(get(w["down"])))

    def forward(self, x, ctx, residual, next_norm=None):
        if self.fused:
            # (a few rows go to the next product k-blocked: it reads them straight from global memory)
            a = ops.linear_swiglu(x, self.w13, blocked_out=True)
        else:
            gu = ops.linear(x, self.w13, torch.float32)
            a = ops.swiglu(gu, self.dtype)
        if next_norm is None:
            ops.linear(a, self.w2, torch.float32, residual=residual)
            return None
        return ops.linear(a, self.w2, torch.float32, residual=residual, next_norm=next_norm)[1]


class GatedFFN(FeedForward):
    """``down(act(gate(x), up(x)))`` with ``act(g, u) = g' * sigmoid(slope * g') * (u' + up_offset)``, where
    g' = min(g, limit) and u' = clamp(u, -limit, limit) when ``limit`` is given.  slope 1, no limit and offset 0 is
    SwiGLU; the constants are parameters of the part.  The activation reads the float32 sums of the gate/up
    product, whatever the compute dtype."""
    graph_safe = True
    returns_output = True      # with ``residual`` None the output comes back instead of being added

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.intermediate_size = int(p["intermediate_size"])
        self.slope = float(p.get("sigmoid_slope", 1.0))
        self.limit = float(p["limit"]) if p.get("limit") is not None else 0.0
        self.up_offset = float(p.get("up_offset", 0.0))
        if self.limit < 0:
            raise ValueError("gated feed-forward: limit must be positive when given")
        self.w13 = None
        self.w2 = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        i, w = spec.params["intermediate_size"], spec.weights
        return {
            w["gate"]: WeightInfo((i, hidden_size)),
            w["up"]: WeightInfo((i, hidden_size)),
            w["down"]: WeightInfo((hidden_size, i)),
        }

    def load_weights(self, get):
        w = self.spec.weights
        gate, up = self._to_device(get(w["gate"])), self._to_device(get(w["up"]))
        # One product.  In bfloat16 the rows alternate eight of gate and eight of up, and the product's epilogue
        # applies the activation to its float32 sums; else gate columns, then up columns, and a kernel of its own.
        self.fused = self.dtype == torch.bfloat16 and ops.gated_layout_ok(self.intermediate_size, self.hidden_size)
        if self.fused:
            self.w13 = ops.tile_weight(ops.interleave_gate_up(gate, up))
        else:
            self.w13 = ops.tile_weight(torch.cat([gate, up], dim=0).contiguous())
        self.w2 = ops.tile_weight(self._to_device(get(w["down"])))

    def forward(self, x, ctx, residual=None):
        if self.fused and x.shape[0] >= ops.gated_epilogue_rows:
            a = ops.linear_swiglu(x, self.w13, slope=self.slope, limit=self.limit, up_offset=self.up_offset)
        else:
            # (a few rows, or sizes the fused product does not take: the product's float32 sums, then the activation)
            gu = ops.linear(x, self.w13, torch.float32)
            a = ops.gated_act(gu, self.dtype, self.slope, self.limit, self.up_offset, interleaved=self.fused)
        return ops.linear(a, self.w2, torch.float32, residual=residual)


register_part("ffn", "swiglu", SwiGLU)
register_part("ffn", "gated", GatedFFN)
