"""Combiners: what goes on to the next block where that is not the block's own result.

Depth average: with X_0 the stream as the first such block receives it and X_(i+1) the result of
the i-th, the stream that leaves block i is sum_{j <= i + 1} w_i[j] X_j with learned numbers w_i, in
32-bit and in the order of j.  Every block's result is kept for the rest of the step (rows x width x 4
bytes a block)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Combiner, register_combiner

_KEY = ("depth_average", "results")


@register_combiner("depth_average")
class DepthAverage(Combiner):
    """params: inputs (how many results the sum runs over: the block's place among the averaging
    blocks + 2), weight (tensor name, `[inputs]`)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.inputs, self.name = int(spec.params["inputs"]), spec.params["weight"]
        if self.inputs < 2:
            raise ValueError(f"depth_average: a sum over {self.inputs} results; the first block's runs over 2")
        self.weight = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.inputs,), init="ones")}

    def load(self, get):
        self.weight = get(self.name).to(torch.float32).contiguous()

    def enter(self, h, ctx):
        results = ctx._memo.setdefault(_KEY, [])
        if self.inputs == 2:
            del results[:]
        if not results:
            results.append(h)                    # X_0 stays as it is: the block works on a copy
            work = torch.empty_like(h)
            work.copy_(h)
            return work
        return h                                 # the sum the block before made: nobody else holds it

    def leave(self, h, ctx, keep_rows=None):
        results = ctx._memo[_KEY]
        if len(results) + 1 != self.inputs:
            raise RuntimeError(f"depth_average: {len(results) + 1} results at a block whose sum runs over {self.inputs}")
        results.append(h)
        out = torch.empty_like(h)
        # earlier results hold all rows of the step; the last one was reduced to the wanted rows
        if keep_rows is not None:
            ops.weighted_sum(results, self.weight, out, row_idx=keep_rows, n_indexed=len(results) - 1)
        else:
            ops.weighted_sum(results, self.weight, out)
        return out
