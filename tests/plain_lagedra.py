"""A plain, slow implementation of the Lagedra decoder in numpy float64, one function per
mechanism, written from the design's equations and sharing no code with the product path.

The design: the token's row of the table plus a learned row for its position; layers with two
parallel branches off the same input, x + mixer(n1(x)) + ff(n2(x)), where a norm is an RMS norm
with one gain for the whole vector; after every layer the stream that goes on is a learned
weighted sum of the embedding output and all layer results so far; a mixer is linear attention
with a per-head decay ("lightning") or windowed softmax attention with short convolutions, a
partial half-split rotation, per-head temperatures, capped scores and values blended with an
earlier layer's; a feed-forward is dense (gelu) or a mixture of clamped gated experts with a
router that first keeps the best groups of neighbouring experts.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ------------------------------------------------------------------ file reading
def read_safetensors(path: str):
    """name -> float64 array (int32 for integer tables): header length, JSON header, raw data."""
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        head = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, e in head.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = data[lo:hi]
        if e["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif e["dtype"] == "F32":
            a = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif e["dtype"] == "I32":
            a = np.frombuffer(raw, dtype="<i4").copy()
        else:
            raise ValueError(f"{name}: dtype {e['dtype']}")
        out[name] = a.reshape(e["shape"])
    return out


# ------------------------------------------------------------------ small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def scalar_rms_norm(x, g: float, eps: float):
    """x / sqrt(mean(x^2) + eps) times one number."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * g


def rms_norm(x, w, eps: float):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w


# ------------------------------------------------------------------ feed-forwards
def dense_ffn(h, up, down):
    return gelu_tanh(h @ up.T) @ down.T


def expert(h, gate, up, down, limit: float):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(z, top: int, n_groups: int, keep: int):
    """z [experts] router logits of one token -> (chosen experts, their weights).  Scores are the
    softmax over all experts; the experts form `n_groups` groups of neighbours, a group's score is
    its best expert's, only experts of the `keep` best groups can be chosen; the weights are the
    chosen scores over their sum."""
    e = np.exp(z - z.max())
    s = e / e.sum()
    per = len(s) // n_groups
    group_score = s.reshape(n_groups, per).max(axis=1)
    kept = np.argsort(-group_score, kind="stable")[:keep]
    allowed = np.zeros(len(s), dtype=bool)
    for g in kept:
        allowed[g * per:(g + 1) * per] = True
    masked = np.where(allowed, s, -1.0)
    chosen = np.argsort(-masked, kind="stable")[:top]
    w = s[chosen] / (s[chosen].sum() + 1e-20)
    return chosen, w


def route_margin(z, top: int, n_groups: int, keep: int) -> float:
    """How far the router's decision for one token is from going the other way: the smallest gap, in
    logits, between what was just taken and what was just left out (the last kept group against the
    best group left out, the last chosen expert against the best one left out among the kept groups).
    Infinite where nothing is left out.  A run in reduced precision may decide a token with a small
    margin differently; a comparison passes such tokens over."""
    per = len(z) // n_groups
    gz = np.sort(z.reshape(n_groups, per).max(axis=1))[::-1]
    margin = gz[keep - 1] - gz[keep] if keep < n_groups else math.inf
    kept = np.argsort(-z.reshape(n_groups, per).max(axis=1), kind="stable")[:keep]
    allowed = np.sort(np.concatenate([z[g * per:(g + 1) * per] for g in kept]))[::-1]
    if top < len(allowed):
        margin = min(margin, allowed[top - 1] - allowed[top])
    return float(margin)


def moe_ffn(h, w, m, margins=None, forced=None, choices=None):
    """h [t][width]; w: tensors of the feed-forward ("router", "e<i>.gate" ...); m: its config.
    `margins`, a list, gets every token's `route_margin`, `choices`, a list, the router's own choices
    [t][top].  `forced` [t][top]: the experts to take instead
    of the router's own choice (their weights are still their scores over the sum of their scores), for
    a comparison with a run that decided a close call the other way."""
    r = m["router"]
    z = h @ w["router"].T
    out = np.zeros_like(h)
    if margins is not None:
        margins.append(np.array([route_margin(z[t], r["top"], r["groups"]["count"], r["groups"]["keep"])
                                 for t in range(h.shape[0])]))
    own = []
    for t in range(h.shape[0]):
        chosen, weights = route(z[t], r["top"], r["groups"]["count"], r["groups"]["keep"])
        own.append(chosen)
        if forced is not None:
            chosen = np.asarray(forced[t])
            sc = np.exp(z[t] - z[t].max())
            sc = sc / sc.sum()
            weights = sc[chosen] / (sc[chosen].sum() + 1e-20)
        for e, wt in zip(chosen, weights):
            out[t] += wt * expert(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], m["expert"]["limit"])
    if choices is not None:
        choices.append(np.stack(own))
    return out


# ------------------------------------------------------------------ lightning attention
def lightning(h, w, m, eps: float, state=None):
    """h [t][width] of one sequence -> (output [t][width], state [heads][dim][vdim]).
    S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head; the heads side by side are RMS-normed
    with a gain vector, gated by sigmoid(Wg h) and projected."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ w["q"].T).reshape(T, H, D)
    k = silu(h @ w["k"].T).reshape(T, H, D)
    v = silu(h @ w["v"].T).reshape(T, H, V)
    S = np.zeros((H, D, V)) if state is None else state.copy()
    o = np.zeros((T, H, V))
    for t in range(T):
        for hd in range(H):
            S[hd] = m["decay"][hd] * S[hd] + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    y = rms_norm(o.reshape(T, H * V), w["norm"], eps) * sigmoid(h @ w["g"].T)
    return y @ w["o"].T, S


# ------------------------------------------------------------------ attention
def causal_conv(u, w, before=None):
    """u [t][channels], w [channels][taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros (or the
    rows `before`, the sequence's last taps - 1 inputs) ahead of the first row."""
    taps = w.shape[1]
    pad = np.zeros((taps - 1, u.shape[1])) if before is None else before
    full = np.concatenate([pad, u], axis=0)
    y = np.zeros_like(u)
    for j in range(taps):
        y += w[:, j] * full[j:j + u.shape[0]]
    return y, full[full.shape[0] - (taps - 1):]


def yarn_frequencies(dims: int, base: float, scaling):
    """f_i = base^(-2i/dims), i < dims/2, blended towards f_i / factor over a ramp between the pair
    indices where `fast` and `slow` turns fit into `original` positions; (frequencies, magnitude)."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index(scaling["fast"])), 0)
    hi = min(math.ceil(index(scaling["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, dims: int, base: float, scaling):
    """x [t][heads][d]: value i < dims/2 is paired with value i + dims/2; values from `dims` on pass."""
    f, mag = yarn_frequencies(dims, base, scaling)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    c, s = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
    half = dims // 2
    a, b = x[..., :half], x[..., half:dims]
    return np.concatenate([a * c - b * s, b * c + a * s, x[..., dims:]], axis=-1)


def windowed_attention(h, w, m, v_first=None):
    """h [t][width] of one whole sequence from position 0 -> (output [t][width], this layer's
    values before any blending [t][kv_heads][vdim])."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    if m.get("conv"):
        q, k, v = causal_conv(q, w["q.conv"])[0], causal_conv(k, w["k.conv"])[0], causal_conv(v, w["v.conv"])[0]
    q, k, v = q.reshape(T, H, D), k.reshape(T, G, D), v.reshape(T, G, V)
    rot = m.get("rot")
    if rot:
        pos = np.arange(T)
        q = rotate_half(q, pos, rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate_half(k, pos, rot["dims"], rot["base"], rot.get("scaling"))
    own = v
    if v_first is not None:
        lam = float(np.asarray(w["vmix"]).reshape(()))
        v = (1.0 - lam) * v + lam * v_first
    window = (m.get("mask") or {}).get("size")
    cap = m.get("softcap")
    o = np.zeros((T, H, V))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] * float(w["temp"][hd])
        if cap:
            s = cap * np.tanh(s / cap)
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        seen = (j <= i) if window is None else ((j <= i) & (i - j < window))
        s = np.where(seen, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        o[:, hd] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g]
    return o.reshape(T, H * V) @ w["o"].T, own


# ------------------------------------------------------------------ the model
class PlainLagedra:
    def __init__(self, config: dict, tensors: dict):
        self.c, self.w = config, tensors

    @classmethod
    def from_folder(cls, folder: str):
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        return cls(config, read_safetensors(os.path.join(folder, "model.safetensors")))

    def sub(self, prefix: str):
        return {n[len(prefix):]: t for n, t in self.w.items() if n.startswith(prefix)}

    def forward(self, tokens, layers_out=None, margins=None, routes=None, choices=None):
        """Logits [t][vocab] of one sequence from position 0.  `layers_out`, a list, gets the stream
        that leaves every layer; `margins`, a list, one array of `route_margin` per routed layer;
        `routes`: layer number -> [t][top] experts to take in that layer, `choices`, a list, one array
        [t][top] of the router's own choices per routed layer (`moe_ffn`)."""
        c, w = self.c, self.w
        eps = c["norm"]["eps"]
        T = len(tokens)
        x = w["embed"][np.asarray(tokens)] + w["pos"][:T]
        results = [x]
        v_first = None
        for i, layer in enumerate(c["layers"]):
            p = f"l{i}."
            a = scalar_rms_norm(x, float(w[p + "norm1"].reshape(())), eps)
            m = layer["mixer"]
            if layer["type"] == "lightning":
                y = lightning(a, self.sub(p + "mix."), m, eps)[0]
            else:
                mixes = bool(m.get("v_mix"))
                y, own = windowed_attention(a, self.sub(p + "mix."), m, v_first if mixes else None)
                if mixes and v_first is None:
                    v_first = own
            if layer["mlp"] is not None:
                b = scalar_rms_norm(x, float(w[p + "norm2"].reshape(())), eps)
                mw = self.sub(p + "mlp.")
                y = y + (dense_ffn(b, mw["up"], mw["down"]) if layer["mlp"]["kind"] == "dense"
                         else moe_ffn(b, mw, layer["mlp"], margins, None if routes is None else routes.get(i), choices))
            results.append(x + y)
            x = sum(w[p + "dwa"][j] * results[j] for j in range(i + 2))
            if layers_out is not None:
                layers_out.append(x)
        return scalar_rms_norm(x, float(w["final.norm"].reshape(())), eps) @ w["head"].T


    def routed_layers(self):
        return [i for i, layer in enumerate(self.c["layers"]) if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe"]


def greedy(logits_row) -> int:
    return int(np.argmax(logits_row))
