"""Mixture-of-experts feed-forward with a router that first keeps the best groups of experts.

Router: z = Wr x in 32-bit, scores = softmax(z) over all experts; the experts form `groups` equal
groups of neighbours, a group's score is its best expert's, and only experts of the `keep` best groups
can be among the `top` chosen; the chosen experts' scores over their sum are the weights.
Expert (no biases): g = min(Wg x, limit), u = clamp(Wu x, -limit, limit), y = g sigmoid(1.702 g) (u + 1),
output Wd y.  The result is the weighted sum of the chosen experts' outputs.

Two forms.  Steps of many tokens run every expert's gate|up over all tokens as one product (the
experts' matrices stacked), apply the activation times the token's weight for the expert (0 where it
was not chosen) and multiply by the experts' down matrices side by side: two products whatever
the routing, experts / top times the arithmetic of the chosen experts alone.  Steps of few tokens
read only the chosen experts' matrices (`ops.moe_sparse`).

A step whose context carries a list under `_memo["route_log"]` gets every routed layer's choices
(`[rows][top]` expert numbers, on the device) appended to it, in run order.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, register_feed_forward
from .linear import Linear

# steps of at most this many tokens read only the chosen experts' matrices
SPARSE_UP_TO = ops.MOE_SPARSE_TOKENS


@register_feed_forward("grouped_moe")
class GroupedMoE(FeedForward):
    """params: hidden_size, intermediate_size (of one expert), n_experts, top, groups, keep, limit,
    router (tensor name), expert (format of an expert's tensor stem, e.g. "mlp.e{}"; its matrices are
    stem + ".gate", ".up", ".down")."""

    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter, self.ne, self.top, self.groups, self.keep = (
            int(p[k]) for k in ("hidden_size", "intermediate_size", "n_experts", "top", "groups", "keep"))
        self.limit = float(p["limit"])
        self.router_name, self.expert_name = p["router"], p["expert"]
        per = self.ne // max(1, self.groups)
        if self.ne % self.groups or not 1 <= self.keep <= self.groups or not 1 <= self.top <= min(64, self.keep * per) \
                or self.ne > ops.MOE_MAX_EXPERTS:
            raise ValueError(f"grouped_moe: {self.ne} experts in {self.groups} groups, {self.keep} kept, {self.top} chosen")
        self.router = self.gate_up = self.down = None

    def tensor_specs(self):
        s = {self.router_name: TensorSpec((self.ne, self.hidden))}
        for e in range(self.ne):
            stem = self.expert_name.format(e)
            s[stem + ".gate"] = TensorSpec((self.inter, self.hidden))
            s[stem + ".up"] = TensorSpec((self.inter, self.hidden))
            s[stem + ".down"] = TensorSpec((self.hidden, self.inter))
        return s

    def load(self, get):
        self.router = get(self.router_name).to(torch.float32).contiguous()   # the router's product is 32-bit
        stems = [self.expert_name.format(e) for e in range(self.ne)]
        rows = []
        for s in stems:
            rows += [get(s + ".gate"), get(s + ".up")]
        self.gate_up = Linear.stacked(rows)                                  # [experts][gate | up][hidden]
        self.down = Linear(torch.cat([get(s + ".down") for s in stems], dim=1).contiguous())   # [hidden][experts x inter]

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return 0

    def forward(self, x, h, ctx, accumulate: bool = True) -> None:
        n, dev = x.shape[0], x.device
        dense = torch.empty((n, self.ne), dtype=torch.float32, device=dev)
        chosen = torch.empty((n, self.top), dtype=torch.int32, device=dev)
        weights = torch.empty((n, self.top), dtype=torch.float32, device=dev)
        ops.moe_route(x, self.router, dense, chosen, weights, self.groups, self.keep)
        log = ctx._memo.get("route_log") if ctx is not None else None
        if log is not None:                  # a caller that wants to know: every routed layer's choices, in run order
            log.append(chosen)
        if n <= SPARSE_UP_TO and n * self.top <= ops.MOE_SPARSE_PAIRS and x.dtype == self.gate_up.weight.dtype:
            if not accumulate:
                h.zero_()
            ops.moe_sparse(x, self.gate_up.weight, self.down.weight, chosen, weights, h, self.ne, self.limit)
            return
        gu = self.gate_up(x, out_dtype=torch.float32)
        y = torch.empty((n, self.ne * self.inter), dtype=self.rt.dtype, device=dev)
        ops.moe_act(gu, dense, y, self.limit)
        self.down(y, out=h, accumulate=accumulate)
