"""Windowed grouped-query attention with keys and values of widths of their own, a short causal
convolution behind the projections, a rotation over part of a head, a temperature per head, capped
scores and values blended with an earlier layer's.

q = Wq x, k = Wk x, v = Wv x (no biases) -> a causal convolution over time on every channel of q, k
and v (`taps` taps, zeros before the sequence's start; the last taps - 1 projected rows of a
sequence are its state) -> the position encoding on q and k -> in a layer that blends,
v <- (1 - lambda) v + lambda v_first with v_first the values (behind their convolution) of the first
layer that names the same `v_share`, same token; the blended v is what is cached -> query head h
reads kv head h // (heads / kv_heads), keys j with 0 <= p - j < window ->
s = cap tanh(q . k scale temp[h] / cap), ordinary softmax, o = sum p_j v_j -> Wo.
"""
from __future__ import annotations

import torch

from ..cache.paged import KVRequest, StateRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, POSITIONS, make_part, register_mixer
from .linear import Linear


@register_mixer("capped_attention")
class CappedAttention(Mixer):
    """params: hidden_size, n_heads, n_kv_heads, dim, v_dim, scale, cap (None or 0: scores are not
    capped), window (None or int), taps (None: no convolution), position (PartSpec of a
    half-split rotation with `half_tables`, or None), v_share (None, or the name under which the
    layers that blend their values find the first one's), v_share_first (True in the first of them),
    q, k, v, o, temp, vmix (tensor names; the convolutions are name + ".conv")."""

    takes_normed = True
    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.nh, self.nk, self.dim, self.vdim = (
            int(p[k]) for k in ("hidden_size", "n_heads", "n_kv_heads", "dim", "v_dim"))
        self.scale = float(p["scale"])
        self.cap = float(p.get("cap") or 0.0)
        self.window = p.get("window")
        self.has_conv = p.get("taps") is not None
        self.taps = int(p["taps"]) if self.has_conv else 1
        self.v_share, self.v_first = p.get("v_share"), bool(p.get("v_share_first", False))
        if self.nh % self.nk:
            raise ValueError(f"capped_attention: {self.nh} heads are not a multiple of {self.nk} kv heads")
        if self.window is not None and int(self.window) < 1:
            raise ValueError(f"capped_attention: window {self.window} must be >= 1")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"capped_attention: {self.taps} taps; the kernels take 1 to {ops.CONV_MAX_TAPS}")
        if self.dim > 512 or self.vdim > 256:
            raise ValueError(f"capped_attention: keys of {self.dim} (at most 512) and values of {self.vdim} (at most 256)")
        self.names = {k: p[k] for k in ("q", "k", "v", "o", "temp", "vmix")}
        self.position = None
        if p.get("position") is not None:
            self.position = make_part(POSITIONS, p["position"], rt, "position encoding")
            if not hasattr(self.position, "half_tables"):
                raise ValueError("capped_attention: the position encoding must be a half-split rotation (half_tables)")
        self.channels = self.nh * self.dim + self.nk * (self.dim + self.vdim)
        self.qkv = self.o = self.conv = self.temp = None
        self.blend = 0.0

    def tensor_specs(self):
        n = self.names
        rows = {"q": self.nh * self.dim, "k": self.nk * self.dim, "v": self.nk * self.vdim}
        s = {n[k]: TensorSpec((r, self.hidden)) for k, r in rows.items()}
        if self.has_conv:
            s.update({n[k] + ".conv": TensorSpec((r, self.taps)) for k, r in rows.items()})
        s[n["o"]] = TensorSpec((self.hidden, self.nh * self.vdim))
        s[n["temp"]] = TensorSpec((self.nh,), init="ones")
        if self.v_share is not None:
            s[n["vmix"]] = TensorSpec(())
        return s

    def load(self, get):
        n = self.names
        self.qkv = Linear.stacked([get(n[k]) for k in ("q", "k", "v")])
        self.o = Linear(get(n["o"]))
        if self.has_conv:
            self.conv = torch.cat([get(n[k] + ".conv").to(torch.float32) for k in ("q", "k", "v")], dim=0).contiguous()
        self.temp = get(n["temp"]).to(torch.float32).contiguous()
        if self.v_share is not None:
            self.blend = float(get(n["vmix"]).to(torch.float32).cpu())      # the first layer's is not used

    def cache_request(self):
        kv = KVRequest(self.nk, self.dim, None if self.window is None else int(self.window),
                       v_head_dim=None if self.vdim == self.dim else self.vdim)
        if self.taps > 1:
            return kv, StateRequest((self.taps - 1, self.channels), torch.float32)
        return kv

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.qkv.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length)

    def prepare(self, max_len: int) -> None:
        if self.position is not None:
            self.position.prepare(max_len)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        kc, vc, group = ctx.cache.kv(entry)
        table = ctx.page_table(group)
        qkv = self.qkv(x, out_dtype=torch.float32)
        n, dev = qkv.shape[0], qkv.device
        cos = sin = None
        if self.position is not None:
            cos, sin = self.position.half_tables(ctx.max_len)
        v_first = v_own = None
        if self.v_share is not None:
            key = ("v_share", self.v_share)
            if self.v_first:
                v_own = ctx._memo[key] = torch.empty((n, self.nk * self.vdim), dtype=torch.float32, device=dev)
            else:
                v_first = ctx._memo.get(key)
                if v_first is None:
                    raise RuntimeError(f"capped_attention: no earlier layer left its values under {self.v_share!r}")
        q = torch.empty((n, self.nh * self.dim), dtype=self.rt.dtype, device=dev)
        ops.qkv_conv_prep(qkv, self.conv, ctx.cache.state(entry) if self.taps > 1 else None, ctx.cu_seqlens,
                          ctx.seq_of_tok, ctx.slot_ids, ctx.positions, cos, sin, self.blend, v_first, v_own, table,
                          q, kc, vc, self.nh, self.nk, self.dim, self.vdim, writes_cache)
        o = torch.empty((n, self.nh * self.vdim), dtype=self.rt.dtype, device=dev)
        window = 0 if self.window is None else int(self.window)
        if ops.capped_mfma_takes(self.rt.dtype, self.dim, self.vdim):
            ops.capped_attn_prefill(q, kc, vc, table, ctx, self.temp, o, self.nh, self.nk, self.dim, self.vdim, self.scale,
                                    self.cap, window)
        else:
            ops.capped_attn(q, kc, vc, table, ctx.positions, ctx.seq_of_tok, self.temp, o, self.nh, self.nk, self.dim,
                            self.vdim, self.scale, self.cap, window, ctx.max_len)
        self.o(o, out=h, accumulate=accumulate)
