"""SwiGLU feed-forward without biases: down( silu(gate x) * (up x) ), silu(z) = z/(1+e^-z)
(src/models/qwen2/graph.rs:154-176, src/graph/cpu_backend.rs:323-329 of yusiwen/minfer).
gate|up are one matrix.  In bfloat16 its rows are interleaved so that the product's epilogue
applies SwiGLU from the 32-bit accumulators and writes y directly; in 32-bit the stacked
product is followed by the SwiGLU kernel.  The down product adds into the residual."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, Normed, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """params: hidden_size, intermediate_size, gate/up/down (tensor name stems)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.names = {k: p[k] for k in ("gate", "up", "down")}
        self.gate_up = self.down = self.fused = self.fused_tiled = None

    def tensor_specs(self):
        n = self.names
        return {n["gate"] + ".weight": TensorSpec((self.inter, self.hidden)),
                n["up"] + ".weight": TensorSpec((self.inter, self.hidden)),
                n["down"] + ".weight": TensorSpec((self.hidden, self.inter))}

    def load(self, get):
        n = self.names
        gate, up = get(n["gate"] + ".weight"), get(n["up"] + ".weight")
        if self.rt.is_bf16 and gate.dtype == up.dtype == torch.bfloat16:
            self.fused = ops.interleave_gate_up(gate, up)
        else:
            self.gate_up = Linear.stacked([gate, up])
        self.down = Linear(get(n["down"] + ".weight"))

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        n = self.down.decode_copy(make, min_row_length)
        if self.fused is not None:
            if self.hidden % 32 == 0 and self.hidden >= min_row_length:
                if make and self.fused_tiled is None:
                    self.fused_tiled = ops.tile_weight(self.fused)
                n += self.fused.numel() * 2
        elif self.gate_up is not None:
            n += self.gate_up.decode_copy(make, min_row_length)
        return n

    takes_normed = True

    def forward(self, x, h, ctx) -> None:
        y = torch.empty((x.shape[0], self.inter), dtype=self.rt.dtype, device=x.device)
        if self.fused is not None:
            fold = x.norm.rms_scale() if isinstance(x, Normed) else None
            done = False
            if fold is not None and x.ahead is not None:      # the product before prepared this norm's input
                done = ops.linear_fused(x.ahead.xg, self.fused, None, y, tiled=self.fused_tiled, swiglu=True,
                                        scale_in=(x.ahead.sums, fold[1]))
            if not done and fold is not None:
                done = ops.linear_normed(x.h, fold[0], fold[1], x.row_idx, self.fused, None, y, swiglu=True,
                                         tiled=self.fused_tiled)
            if not done:
                ops.linear_swiglu(x.tensor() if isinstance(x, Normed) else x, self.fused, y, tiled=self.fused_tiled)
        else:
            ops.swiglu(self.gate_up(x, out_dtype=torch.float32), y)
        self.down(y, out=h, accumulate=True, ctx=ctx)


def _softplus(v: float) -> float:
    import math
    return max(v, 0.0) + math.log1p(math.exp(-abs(v)))


@register_feed_forward("dense_xielu")
class DenseXIELU(FeedForward):
    """down(act(up x + b_up)) + b_down with the xIELU activation: for z > 0, softplus(p) z^2 + z/2;
    for z <= 0, (1/2 + softplus(q)) (e^z - 1 - z) + z/2, where (p, q) are the two values of the
    layer's `act` tensor.  The activation reads the up product's 32-bit sums and is rounded once.
    params: hidden_size, intermediate_size, up, down (tensor names; biases are name + ".b"), act."""

    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.names = {k: p[k] for k in ("up", "down", "act")}
        self.up = self.down = None
        self.a_pos = self.a_neg = None

    def tensor_specs(self):
        n = self.names
        return {n["up"]: TensorSpec((self.inter, self.hidden)), n["up"] + ".b": TensorSpec((self.inter,)),
                n["down"]: TensorSpec((self.hidden, self.inter)), n["down"] + ".b": TensorSpec((self.hidden,)),
                n["act"]: TensorSpec((2,))}

    def load(self, get):
        n = self.names
        self.up = Linear(get(n["up"]), get(n["up"] + ".b"))
        self.down = Linear(get(n["down"]), get(n["down"] + ".b"))
        pq = [float(v) for v in get(n["act"]).to(torch.float32).cpu()]
        self.a_pos, self.a_neg = _softplus(pq[0]), 0.5 + _softplus(pq[1])
        # bfloat16 products apply the activation in their epilogue: its constants ride behind the biases
        self.up_act_bias = None
        if self.rt.is_bf16 and self.up.weight.dtype == torch.bfloat16:
            tail = torch.tensor([self.a_pos, self.a_neg], dtype=torch.float32, device=self.up.bias.device)
            self.up_act_bias = torch.cat([self.up.bias, tail]).contiguous()

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.up.decode_copy(make, min_row_length) + self.down.decode_copy(make, min_row_length)

    def forward(self, x, h, ctx, accumulate: bool = True) -> None:
        y = torch.empty((x.shape[0], self.inter), dtype=self.rt.dtype, device=x.device)
        if self.up_act_bias is not None and x.dtype == torch.bfloat16:
            ops.linear(x, self.up.weight, self.up_act_bias, y, tiled=self.up.tiled, xielu=True)
        else:
            u = self.up(x, out_dtype=torch.float32)
            ops.xielu(u, y, self.a_pos, self.a_neg)
        self.down(y, out=h, accumulate=accumulate)


@register_feed_forward("dense_gelu")
class DenseGelu(FeedForward):
    """down(gelu(up x)) without biases, gelu in its tanh form, from the up product's 32-bit sums and
    rounded once.  params: hidden_size, intermediate_size, up, down (tensor names)."""

    takes_normed = True
    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.names = {k: p[k] for k in ("up", "down")}
        self.up = self.down = None

    def tensor_specs(self):
        n = self.names
        return {n["up"]: TensorSpec((self.inter, self.hidden)), n["down"]: TensorSpec((self.hidden, self.inter))}

    def load(self, get):
        self.up, self.down = Linear(get(self.names["up"])), Linear(get(self.names["down"]))

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.up.decode_copy(make, min_row_length) + self.down.decode_copy(make, min_row_length)

    def forward(self, x, h, ctx, accumulate: bool = True) -> None:
        u = self.up(x, out_dtype=torch.float32)
        y = torch.empty((u.shape[0], self.inter), dtype=self.rt.dtype, device=u.device)
        ops.gelu_tanh(u, y)
        self.down(y, out=h, accumulate=accumulate)
