"""Linear attention with a decay per head ("lightning" attention): a fixed-size matrix state per
sequence and head instead of keys and values.

q = silu(Wq x), k = silu(Wk x) (heads x dim), v = silu(Wv x) (heads x v_dim); per head
S_t = decay_h S_(t-1) + k_t v_t^T from S = 0 at a sequence's start, o_t = S_t^T q_t, no other scale;
the heads side by side are RMS-normed together with a gain vector, multiplied by sigmoid(Wg x) and
projected by Wo.  The state is float32 `[heads][dim][v_dim]` per cache slot; state, decays, products
and sums are 32-bit in both run types.
"""
from __future__ import annotations

import torch

from ..cache.paged import StateRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, register_mixer
from .linear import Linear

# a step whose longest sequence brings more tokens than this walks its sequences in chunks side by side
CHUNKED_FROM = ops.LA_CHUNK


@register_mixer("lightning_attention")
class LightningAttention(Mixer):
    """params: hidden_size, n_heads, dim, v_dim, decays (one number per head), eps (of the norm over
    the heads), q, k, v, g, o, norm (tensor names)."""

    takes_normed = True
    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.nh, self.dim, self.vdim = (int(p[k]) for k in ("hidden_size", "n_heads", "dim", "v_dim"))
        self.eps = float(p["eps"])
        self.decay_values = [float(d) for d in p["decays"]]
        if len(self.decay_values) != self.nh:
            raise ValueError(f"lightning_attention: {len(self.decay_values)} decays for {self.nh} heads")
        if self.dim > 256:
            raise ValueError(f"lightning_attention: key width {self.dim} is beyond what the kernels take (256)")
        self.names = {k: p[k] for k in ("q", "k", "v", "g", "o", "norm")}
        self.proj = self.o = self.norm_weight = self.decays = None

    def tensor_specs(self):
        n, H = self.names, self.nh
        return {n["q"]: TensorSpec((H * self.dim, self.hidden)), n["k"]: TensorSpec((H * self.dim, self.hidden)),
                n["v"]: TensorSpec((H * self.vdim, self.hidden)), n["g"]: TensorSpec((H * self.vdim, self.hidden)),
                n["o"]: TensorSpec((self.hidden, H * self.vdim)), n["norm"]: TensorSpec((H * self.vdim,), init="ones")}

    def load(self, get):
        n = self.names
        self.proj = Linear.stacked([get(n["q"]), get(n["k"]), get(n["v"]), get(n["g"])])     # one product
        self.o = Linear(get(n["o"]))
        self.norm_weight = get(n["norm"]).to(torch.float32).contiguous()
        self.decays = torch.tensor(self.decay_values, dtype=torch.float32, device=self.norm_weight.device)

    def cache_request(self):
        return StateRequest((self.nh, self.dim, self.vdim), torch.float32)

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.proj.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        state = ctx.cache.state(entry)
        proj = self.proj(x, out_dtype=torch.float32)
        n, hv = proj.shape[0], self.nh * self.vdim
        o = torch.empty((n, hv), dtype=torch.float32, device=proj.device)
        chunks = None
        if not ctx.all_decode and ctx.max_new > CHUNKED_FROM and self.dim <= ops.LA_CHUNKED_MAX_DIM:
            key = ("la_chunks",)
            if key not in ctx._memo:
                table, count = ops.la_chunks(ctx.host_new)
                ctx._memo[key] = (table.to(proj.device), count)
            chunks = ctx._memo[key]
        ops.lightning_scan(proj, ctx.cu_seqlens, ctx.slot_ids, self.decays, state, o, self.nh, self.dim, self.vdim, chunks)
        y = torch.empty((n, hv), dtype=self.rt.dtype, device=proj.device)
        ops.gated_rmsnorm(o, proj, 2 * self.nh * self.dim + hv, self.norm_weight, self.eps, y)
        self.o(y, out=h, accumulate=accumulate)
