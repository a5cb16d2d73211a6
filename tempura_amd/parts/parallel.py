"""Several mixers side by side on the same input: the output is sum_i scale_i * mixer_i(x).

The branches are ``BranchMixer`` parts (``branches``: a list of mixer ``PartSpec``; ``scales``: one constant each).
Their input projections are ONE product (the rows of all branches stacked, each branch reading its own columns of
the float32 result) and their output projections are ONE product too: branch i writes scale_i times what enters its
output projection into its own columns of one buffer, and the stacked output weights [hidden, sum of inner sizes]
add the branches up inside the product's sum.  At most one branch keeps pages of the cache; the branches' states
lie one after the other in one float32 row per request.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, StateSpec, build_part, pad_rows, part_class, register_part


class ParallelMixer(Mixer):
    graph_safe = True
    returns_output = True      # with ``residual`` None the output comes back instead of being added

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        specs = list(spec.params["branches"])
        self.scales = [float(v) for v in spec.params.get("scales", [1.0] * len(specs))]
        if not specs or len(self.scales) != len(specs):
            raise ValueError("parallel: one scale per branch, at least one branch")
        self.branches = [build_part("mixer", ps, hidden_size, dtype, device) for ps in specs]
        for b in self.branches:
            if not hasattr(b, "load_branch"):
                raise ValueError(f"parallel: mixer {b.spec.kind!r} cannot share its products (no load_branch)")
        if sum(b.cache_spec() is not None for b in self.branches) > 1:
            raise ValueError("parallel: at most one branch may keep pages of the cache")
        off = 0
        for b in self.branches:
            b.state_off = off
            off += b.state_floats()
        self.state_total = off
        self.graph_safe = all(b.graph_safe for b in self.branches)
        self.preferred_portion_align = max(int(getattr(b, "preferred_portion_align", 1)) for b in self.branches)
        self.inner = sum(b.inner for b in self.branches)
        self.w_in = self.w_out = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        out = {}
        for ps in spec.params["branches"]:
            out.update(part_class("mixer", ps.kind).expected_weights(ps, hidden_size))
        return out

    def load_weights(self, get):
        ins, outs = [], []
        self.in_cols, self.out_cols = [], []
        col = ocol = 0
        for b in self.branches:
            w_in, w_out = b.load_branch(get)
            ins.append(w_in)
            outs.append(w_out)
            self.in_cols.append(col)
            self.out_cols.append(ocol)
            col += w_in.shape[0]
            ocol += w_out.shape[1]
        self.w_in = ops.tile_weight(pad_rows(torch.cat(ins, dim=0), 16))
        self.w_out = ops.tile_weight(torch.cat(outs, dim=1).contiguous())

    def cache_spec(self):
        for b in self.branches:
            cs = b.cache_spec()
            if cs is not None:
                return cs
        return None

    def state_spec(self):
        return StateSpec((self.state_total,), torch.float32) if self.state_total else None

    def forward(self, x, ctx, cache, residual=None):
        proj = ops.linear(x, self.w_in, torch.float32)
        act = torch.empty((proj.shape[0], self.inner), dtype=self.dtype, device=proj.device)
        for b, scale, col, ocol in zip(self.branches, self.scales, self.in_cols, self.out_cols):
            b.run(proj, col, ctx, cache, act, ocol, scale)
        return ops.linear(act, self.w_out, torch.float32, residual=residual)


register_part("mixer", "parallel", ParallelMixer)
