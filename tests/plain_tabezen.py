"""A plain, slow implementation of the Tabezen decoder in numpy float64, one function per
mechanism, written from the design's equations and sharing no code with the product path.

The design: the token's row of the table, normed; layers h <- h + N1(mixer(h)) and then
h <- h + N2(ff(h)), where the branches read the stream itself and only their results are normed;
a final norm and the output matrix.  N is an RMS norm taken over `groups` equal consecutive parts
of the vector.  A mixer is a minGRU recurrence or attention over a shared low-rank latent with a
rotated key part of its own.  A layer may borrow another layer's tensors.
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


def softplus(z):
    return np.logaddexp(0.0, z)


def silu(z):
    return z * sigmoid(z)


def group_rms_norm(x, w, eps: float, groups: int):
    """x [..., d]: each of `groups` consecutive parts over its own sqrt(mean(part^2) + eps), all times w."""
    d = x.shape[-1]
    parts = x.reshape(x.shape[:-1] + (groups, d // groups))
    y = parts / np.sqrt((parts * parts).mean(axis=-1, keepdims=True) + eps)
    return y.reshape(x.shape) * w


def xielu(z, p: float, q: float):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (np.expm1(np.minimum(z, 0.0)) - z) + 0.5 * z
    return np.where(z > 0, pos, neg)


def dense_ffn(h, up, up_b, down, down_b, act):
    return xielu(h @ up.T + up_b, float(act[0]), float(act[1])) @ down.T + down_b


# ------------------------------------------------------------------ rotation
def yarn_frequencies(dims: int, base: float, scaling):
    """f_i = base^(-2i/dims) for the pairs i < dims/2, blended towards f_i / factor over a ramp
    between the pair indices where `fast` and `slow` turns fit into `original` positions; returns
    the frequencies and the factor that cos and sin are multiplied by."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, dims: int, base: float, scaling):
    """x [t, ..., n]: the first `dims` values of the last axis are rotated in pairs (2i, 2i+1) by
    the angle position * f_i; the rest pass unchanged."""
    f, mag = yarn_frequencies(dims, base, scaling)
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (dims // 2,)
    ang = (np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]).reshape(shape)
    c, s = np.cos(ang) * mag, np.sin(ang) * mag
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------ mixers
def mingru(h, w, state=None):
    """z = sigmoid(Wz h + bz); u = Wx h + bx; cand = u + 1/2 (u >= 0), sigmoid(u) (u < 0);
    S_t = (1 - z) S_(t-1) + z cand; out = Wo (S_t silu(Wg h)).  Returns (out, last state)."""
    z = sigmoid(h @ w["z"].T + w["z.b"])
    u = h @ w["x"].T + w["x.b"]
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    g = silu(h @ w["g"].T)
    s = np.zeros(z.shape[1]) if state is None else state.copy()
    rows = np.empty_like(z)
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        rows[t] = s
    return (rows * g) @ w["o"].T, s


def latent_attention(h, w, m, eps: float, positions=None):
    """Queries per head [dim plain | rot_dim rotated]; one latent c = rmsnorm(first kv_rank rows
    of Wdkv h) and one rotated key part (the last rot_dim rows) for all heads; per head
    k = Wuk c, v = Wuv c; softmax over j <= i of (q_plain . k + q_rot . k_rot) scale; each head's
    result times sigmoid(Wg h)_head; then Wo."""
    t = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    pos = np.arange(t) if positions is None else np.asarray(positions)
    q = (h @ w["q"].T).reshape(t, H, dn + dr)
    q_plain = q[:, :, :dn]
    q_rot = rotate_interleaved(q[:, :, dn:], pos, rot["dims"], rot["base"], rot.get("scaling"))
    dkv = h @ w["dkv"].T
    c = dkv[:, :r]
    c = c / np.sqrt((c * c).mean(axis=-1, keepdims=True) + eps) * w["dkv.norm"]
    k_rot = rotate_interleaved(dkv[:, r:], pos, rot["dims"], rot["base"], rot.get("scaling"))
    k = (c @ w["uk"].T).reshape(t, H, dn)
    v = (c @ w["uv"].T).reshape(t, H, dv)
    gate = sigmoid(h @ w["g"].T)                       # [t, H]
    out = np.zeros((t, H, dv))
    for hd in range(H):
        s = (q_plain[:, hd] @ k[:, hd].T + q_rot[:, hd] @ k_rot.T) * m["scale"]
        s = np.where(pos[None, :] <= pos[:, None], s, -np.inf)
        s = s - s.max(axis=-1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=-1, keepdims=True)
        out[:, hd] = (p @ v[:, hd]) * gate[:, hd:hd + 1]
    return out.reshape(t, H * dv) @ w["o"].T


# ------------------------------------------------------------------ the model
class PlainTabezen:
    def __init__(self, config: dict, tensors: dict):
        self.cfg, self.t = config, tensors
        self.eps, self.groups = float(config["norm"]["eps"]), int(config["norm"]["groups"])

    @classmethod
    def from_folder(cls, folder: str):
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, read_safetensors(os.path.join(folder, "model.safetensors")))

    def norm(self, x, name):
        return group_rms_norm(x, self.t[name], self.eps, self.groups)

    def layer_tensors(self, i: int, part: str):
        owner = self.cfg["layers"][i].get("weights_of", i)
        owner = i if owner is None else owner
        pre = f"l{owner}.{part}."
        return {k[len(pre):]: v for k, v in self.t.items() if k.startswith(pre)}, f"l{owner}."

    def forward(self, tokens, return_layers: bool = False):
        """All positions' logits [t, vocab] (and the stream after every layer)."""
        x = self.norm(self.t["embed"][np.asarray(tokens)], "embed.norm")
        after = []
        for i, layer in enumerate(self.cfg["layers"]):
            w, pre = self.layer_tensors(i, "mix")
            if layer["type"] == "mingru":
                y, _ = mingru(x, w)
            elif layer["type"] == "latent_attention":
                y = latent_attention(x, w, layer["mixer"], self.eps)
            else:
                raise ValueError(layer["type"])
            x = x + self.norm(y, pre + "norm1")
            if layer.get("mlp"):
                f, _ = self.layer_tensors(i, "mlp")
                x = x + self.norm(dense_ffn(x, f["up"], f["up.b"], f["down"], f["down.b"], f["act"]), pre + "norm2")
            after.append(x.copy())
        logits = self.norm(x, "final.norm") @ self.t["head"].T
        return (logits, np.stack(after)) if return_layers else logits


def greedy(row) -> int:
    return int(np.argmax(row))
