"""A selective state-space mixer in the state-space duality form ("mamba2").

With ``inner = heads * head_dim``, N = ``state_size`` and G = ``groups``, the input projection's columns are
[z: inner | x: inner | B: G N | C: G N | dt: heads].  x, B and C pass a causal convolution per channel
(``conv_taps`` taps, bias) and SiLU.  Per head h (its B and C are those of group h // (heads / G)):

    dt = softplus(dt + dt_bias[h])           a = exp(-exp(a_log[h]) * dt)
    S <- a S + dt * B x^T                    y = S^T C + d[h] * x          (S is [N, head_dim])

y times silu(z) is normed in ``norm_groups`` equal parts, each by its own root mean square, times a weight,
then projected back.  Everything between the two projections is float32 whatever the compute dtype.

Per request the mixer keeps, in one float32 row of the engine's state slots, the convolution's last
``conv_taps - 1`` inputs and the recurrent state; both start at zero and are carried from step to step.  The
kernels find a request's tokens and its row through the step's device tensors, so prompt portions, single decoded
tokens and captured steps run the same launches.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, StateSpec, WeightInfo, register_part


class Mamba2Mixer(Mixer):
    graph_safe = True
    returns_output = True      # with ``residual`` None the output comes back instead of being added

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.state_size = int(p["state_size"])
        self.groups = int(p["groups"])
        self.taps = int(p["conv_taps"])
        self.norm_groups = int(p.get("norm_groups", 1))
        self.norm_eps = float(p["norm_eps"])
        if self.num_heads % self.groups != 0:
            raise ValueError("mamba2: heads must be a multiple of groups")
        self.inner = self.num_heads * self.head_dim
        if self.inner % self.norm_groups != 0:
            raise ValueError("mamba2: heads * head_dim must be a multiple of norm_groups")
        self.channels = self.inner + 2 * self.groups * self.state_size      # what the convolution sees: x | B | C
        self.proj_dim = 2 * self.inner + 2 * self.groups * self.state_size + self.num_heads
        self.conv_state = (self.taps - 1) * self.channels
        self.w_in = self.w_out = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        heads, inner = p["num_heads"], p["num_heads"] * p["head_dim"]
        channels = inner + 2 * p["groups"] * p["state_size"]
        return {
            w["in"]: WeightInfo((2 * inner + 2 * p["groups"] * p["state_size"] + heads, hidden_size)),
            w["conv"]: WeightInfo((channels, p["conv_taps"])),
            w["conv_bias"]: WeightInfo((channels,)),
            w["dt_bias"]: WeightInfo((heads,)),
            w["a_log"]: WeightInfo((heads,)),
            w["d"]: WeightInfo((heads,)),
            w["norm"]: WeightInfo((inner,), "ones"),
            w["out"]: WeightInfo((hidden_size, inner)),
        }

    def load_weights(self, get):
        w = self.spec.weights
        w_in = self._to_device(get(w["in"]))
        # rows padded to a multiple of 16 (zeros): the products then take the weight in their tiled form; the
        # kernels behind read the projection's rows by their stride and never see the padding
        pad = (-w_in.shape[0]) % 16
        if pad:
            w_in = torch.cat([w_in, torch.zeros((pad, w_in.shape[1]), dtype=w_in.dtype, device=w_in.device)], dim=0).contiguous()
        self.w_in = ops.tile_weight(w_in)
        f32 = lambda name: self._to_device(get(w[name]), torch.float32)
        self.conv_w, self.conv_b = f32("conv").t().contiguous(), f32("conv_bias")      # (tap-major for the kernel)
        self.dt_bias, self.a_log, self.d_skip = f32("dt_bias"), f32("a_log"), f32("d")
        self.norm_w = f32("norm")
        self.w_out = ops.tile_weight(self._to_device(get(w["out"])))

    def state_spec(self):
        return StateSpec((self.conv_state + self.num_heads * self.state_size * self.head_dim,), torch.float32)

    def forward(self, x, ctx, cache, residual=None):
        proj = ops.linear(x, self.w_in, torch.float32)                  # [n, z | x | B | C | dt (| padding)]
        xbc = ops.causal_conv(proj, self.inner, self.channels, self.conv_w, self.conv_b, cache.state, ctx.cu_seqlens,
                              ctx.token_req, ctx.state_slots, ctx.num_requests)
        y = ops.ssm_scan(xbc, proj, self.inner + self.channels, self.dt_bias, self.a_log, self.d_skip, cache.state,
                         self.conv_state, ctx.cu_seqlens, ctx.state_slots, ctx.num_requests, self.num_heads, self.head_dim,
                         self.state_size, self.groups, max_run=ctx.max_q_len)
        v = ops.gated_group_norm(y, proj, 0, self.norm_w, self.norm_eps, self.norm_groups, self.dtype)
        return ops.linear(v, self.w_out, torch.float32, residual=residual)


register_part("mixer", "mamba2", Mamba2Mixer)
