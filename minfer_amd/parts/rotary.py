"""Rotary position encodings.

Half-split ("NeoX") rotary position encoding over the whole head: element i pairs with
i + head_dim/2, angle = position * freq_scale / theta^(2i/head_dim)
(src/graph/cpu_backend.rs:403-434 of yusiwen/minfer; q and k are rotated after their bias
and before the cache write, v is not, src/models/qwen2/graph.rs:100-113).  cos and sin come
from a table built once on the device in double precision.  The attention mixer takes the
tables and rotates inside its own kernels; `encode` is the plain form for any other user."""
from __future__ import annotations

from ..kernels import ops
from .base import PositionEncoding, register_position

# positions the table is first built for; it doubles from there up to the model's bound, and a
# table that covers the bound is never replaced (so a captured step's address stays good)
FIRST_TABLE = 4096


@register_position("rope_neox")
class RotaryNeoX(PositionEncoding):
    """params: head_dim, theta, max_positions, freq_scale (default 1)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.head_dim, self.theta = int(p["head_dim"]), float(p["theta"])
        self.freq_scale = float(p.get("freq_scale", 1.0))
        self.max_positions = int(p["max_positions"])
        if self.head_dim % 2:
            raise ValueError(f"rope_neox: head_dim {self.head_dim} is odd")
        self.cos = self.sin = None
        self.generation = 0            # moves on when the table is replaced by a longer one

    def prepare(self, max_len: int) -> None:
        if max_len > self.max_positions:
            raise ValueError(f"position {max_len - 1} is beyond the model's {self.max_positions} positions")
        have = 0 if self.cos is None else self.cos.shape[0]
        if max_len > have:
            n = min(self.max_positions, max(FIRST_TABLE, 1 << (max_len - 1).bit_length()))
            if self.cos is not None:
                self.generation += 1
                ops.note_replaced_buffer(self.cos)
                ops.note_replaced_buffer(self.sin)
            self.cos, self.sin = ops.rope_table(n, self.head_dim // 2, self.theta, self.freq_scale,
                                                self.rt.device)

    def rotation_tables(self, max_len: int):
        self.prepare(max_len)
        return self.cos, self.sin

    def encode(self, qkv, ctx, n_heads: int, n_kv_heads: int) -> None:
        self.prepare(ctx.max_len)
        ops.rope_inplace(qkv, self.cos, self.sin, ctx.positions, n_heads + n_kv_heads,
                         n_heads + 2 * n_kv_heads, self.head_dim)


def blended_frequencies(dims: int, base: float, scaling=None):
    """(frequencies of the dims/2 pairs, magnitude).  f_i = base^(-2i/dims).  With `scaling` =
    dict(factor, original, fast, slow) the ladder is stretched for contexts longer than `original`
    positions: pairs that turn more than `fast` times over `original` positions keep f_i, pairs that
    turn fewer than `slow` times get f_i / factor, and the pairs between are blended linearly in the
    pair index: with pair(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(pair(fast)), 0),
    hi = min(ceil(pair(slow)), dims - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i); cos and sin are then multiplied by
    0.1 ln(factor) + 1."""
    import math
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
    lo = max(math.floor(pair(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


@register_position("rope_pairs")
class RotaryPairs(PositionEncoding):
    """Rotation in neighbouring pairs: value 2i with 2i+1, i < dims/2, by the angle position * f_i;
    what lies behind the first `dims` values of a head passes unchanged.  The frequency ladder is
    `blended_frequencies` (plain without `scaling`).  params: dims, base, scaling (None or the
    dict above), max_positions.  `pair_tables` hands the tables to a mixer that rotates inside its
    own kernels; `encode` is the plain form on q|k|v rows."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.dims, self.base = int(p["dims"]), float(p["base"])
        self.scaling = p.get("scaling")
        self.max_positions = int(p["max_positions"])
        if self.dims % 2 or self.dims < 2:
            raise ValueError(f"rope_pairs: {self.dims} rotated values do not form pairs")
        self.freqs, self.magnitude = blended_frequencies(self.dims, self.base, self.scaling)
        self.cos = self.sin = None

    def prepare(self, max_len: int) -> None:
        if max_len > self.max_positions:
            raise ValueError(f"position {max_len - 1} is beyond the model's {self.max_positions} positions")
        have = 0 if self.cos is None else self.cos.shape[0]
        if max_len > have:
            n = min(self.max_positions, max(FIRST_TABLE, 1 << (max_len - 1).bit_length()))
            if self.cos is not None:
                ops.note_replaced_buffer(self.cos)
                ops.note_replaced_buffer(self.sin)
            self.cos, self.sin = ops.rope_table_freqs(n, self.freqs, self.magnitude, self.rt.device)

    def pair_tables(self, max_len: int):
        self.prepare(max_len)
        return self.cos, self.sin

    def encode(self, qkv, ctx, n_heads: int, n_kv_heads: int) -> None:
        self.prepare(ctx.max_len)
        total = n_heads + 2 * n_kv_heads
        ops.rope_pairs_inplace(qkv, self.cos, self.sin, ctx.positions, n_heads + n_kv_heads, total,
                               qkv.shape[1] // total)


@register_position("rope_half")
class RotaryHalf(PositionEncoding):
    """Half-split rotation over the first `dims` values of a head: value i < dims/2 turns with value
    i + dims/2 by the angle position * f_i; what lies behind the first `dims` values passes unchanged.
    The frequency ladder is `blended_frequencies` (plain without `scaling`).  params: dims, base, scaling
    (None or dict(factor, original, fast, slow)), max_positions.  `half_tables` hands the tables
    `[positions][dims / 2]` to a mixer that rotates inside its own kernels; `encode` is the plain form."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.dims, self.base = int(p["dims"]), float(p["base"])
        self.scaling = p.get("scaling")
        self.max_positions = int(p["max_positions"])
        if self.dims % 2 or self.dims < 2:
            raise ValueError(f"rope_half: {self.dims} rotated values do not form pairs")
        self.freqs, self.magnitude = blended_frequencies(self.dims, self.base, self.scaling)
        self.cos = self.sin = None

    def prepare(self, max_len: int) -> None:
        if max_len > self.max_positions:
            raise ValueError(f"position {max_len - 1} is beyond the model's {self.max_positions} positions")
        have = 0 if self.cos is None else self.cos.shape[0]
        if max_len > have:
            n = min(self.max_positions, max(FIRST_TABLE, 1 << (max_len - 1).bit_length()))
            if self.cos is not None:
                ops.note_replaced_buffer(self.cos)
                ops.note_replaced_buffer(self.sin)
            self.cos, self.sin = ops.rope_table_freqs(n, self.freqs, self.magnitude, self.rt.device)

    def half_tables(self, max_len: int):
        self.prepare(max_len)
        return self.cos, self.sin

    def encode(self, qkv, ctx, n_heads: int, n_kv_heads: int) -> None:
        self.prepare(ctx.max_len)
        total = n_heads + 2 * n_kv_heads
        ops.rope_half_inplace(qkv, self.cos, self.sin, ctx.positions, n_heads + n_kv_heads, total, qkv.shape[1] // total)
