"""Recurrent mixers: a fixed-size state per sequence instead of keys and values.

minGRU: z = sigmoid(Wz x + bz), u = Wx x + bx, candidate c = u + 1/2 where u >= 0 and sigmoid(u)
where u < 0; element by element S_t = (1 - z_t) S_(t-1) + z_t c_t from S = 0 at a sequence's
start; the output is Wo (S_t * silu(Wg x)).  The gates read the current token only, so a prompt's
states follow from a scan over its tokens.  The state is float32 `[width]` per cache slot.
"""
from __future__ import annotations

import torch

from ..cache.paged import StateRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, register_mixer
from .linear import Linear

# a step whose longest sequence brings more tokens than this walks its sequences in chunks side by side
CHUNKED_FROM = 2 * ops.SCAN_CHUNK


@register_mixer("mingru")
class MinGRU(Mixer):
    """params: hidden_size, width, z, x, g, o (tensor names; the biases of z and x are name + ".b")."""

    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.width = int(p["hidden_size"]), int(p["width"])
        self.names = {k: p[k] for k in ("z", "x", "g", "o")}
        self.zug = self.o = None

    def tensor_specs(self):
        n = self.names
        return {n["z"]: TensorSpec((self.width, self.hidden)), n["z"] + ".b": TensorSpec((self.width,)),
                n["x"]: TensorSpec((self.width, self.hidden)), n["x"] + ".b": TensorSpec((self.width,)),
                n["g"]: TensorSpec((self.width, self.hidden)),
                n["o"]: TensorSpec((self.hidden, self.width))}

    def load(self, get):
        n = self.names
        self.zug = Linear.stacked([get(n["z"]), get(n["x"]), get(n["g"])],
                                  [get(n["z"] + ".b"), get(n["x"] + ".b"), None])
        self.o = Linear(get(n["o"]))

    def cache_request(self):
        return StateRequest((self.width,), torch.float32)

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.zug.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        state = ctx.cache.state(entry)
        zug = self.zug(x, out_dtype=torch.float32)
        y = torch.empty((x.shape[0], self.width), dtype=self.rt.dtype, device=x.device)
        chunks = None
        if not ctx.all_decode and ctx.max_new > CHUNKED_FROM:
            key = ("scan_chunks",)
            if key not in ctx._memo:
                ctx._memo[key] = ops.scan_chunks(ctx.host_new).to(x.device)
            chunks = ctx._memo[key]
        ops.mingru_scan(zug, ctx.cu_seqlens, ctx.slot_ids, state, y, chunks)
        self.o(y, out=h, accumulate=accumulate)
