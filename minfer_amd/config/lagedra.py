"""Lagedra: a decoder whose layers run a mixer and a feed-forward side by side off the same input,
each behind an RMS norm with a single gain, and whose stream after every layer is a learned sum of
the embedding output and all layer results so far.  A mixer is linear attention with a decay per
head ("lightning") or windowed softmax attention with short convolutions, a partial rotation,
temperatures per head, capped scores and values blended with the first such layer's; a feed-forward
is dense (gelu) or a mixture of clamped gated experts routed by groups.

config.json: `architecture` = "Lagedra"; `vocab`, `width`, `max_positions`; `norm` = {eps}; `layers`, a
list of {type: "lightning" | "attention", mixer: {...}, mlp: {...} or null}.
Mixer sizes: lightning {heads, dim, vdim, decay: [one per head]}; attention {heads, kv_heads, dim,
vdim, scale, softcap, conv (taps), mask: {size}, rot: {base, dims, scaling: {factor, original, fast,
slow} or null}, v_mix}.  mlp: {kind: "dense", ff} or {kind: "moe", expert: {ff, limit}, router:
{experts, top, groups: {count, keep}}}.
Tensors: embed, pos, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, l<i>.dwa, final.norm, head.
"""
from __future__ import annotations

import copy
import math
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError, KeyReader
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, straight_schedule

ARCHITECTURE = "Lagedra"
MIXER_TYPES = ("lightning", "attention")
V_SHARE = "v_mix"      # the name under which the layers that blend their values find the first one's


def _mixer_sizes(kind: str, raw: Any, where: str) -> Dict[str, Any]:
    r = KeyReader(raw, where)
    if kind == "lightning":
        out = dict(heads=r.integer("heads"), dim=r.integer("dim"), vdim=r.integer("vdim"))
        decay = r.raw_value("decay")
        if not isinstance(decay, list) or len(decay) != out["heads"] or \
                any(isinstance(d, bool) or not isinstance(d, (int, float)) or not 0.0 <= d <= 1.0 for d in decay):
            raise ConfigError(f"{where}: 'decay' must list one number in [0, 1] per head, found {decay!r}")
        out["decay"] = [float(d) for d in decay]
        return out
    out = dict(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
               scale=r.number("scale"))
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{where}: 'heads' {out['heads']} is not a multiple of 'kv_heads' {out['kv_heads']}")
    cap = r.raw_value("softcap")
    out["softcap"] = None if cap is None else r.number("softcap")
    out["conv"] = r.integer("conv", default=None)
    mask = r.raw_value("mask")
    out["mask"] = None if mask is None else dict(size=KeyReader(mask, where + ".mask").integer("size"))
    rot = r.raw_value("rot")
    if rot is not None:
        k = KeyReader(rot, where + ".rot")
        dims = k.integer("dims")
        if dims % 2 or dims > out["dim"]:
            raise ConfigError(f"{where}.rot: 'dims' must be even and at most dim {out['dim']}, found {dims}")
        scaling = k.raw_value("scaling")
        if scaling is not None:
            s = KeyReader(scaling, where + ".rot.scaling")
            scaling = dict(factor=s.number("factor"), original=s.number("original"), fast=s.number("fast"),
                           slow=s.number("slow"))
        rot = dict(base=k.number("base"), dims=dims, scaling=scaling)
    out["rot"] = rot
    out["v_mix"] = r.boolean("v_mix", default=False)
    return out


def _mlp_sizes(raw: Any, where: str) -> Optional[Dict[str, Any]]:
    if raw is None:
        return None
    m = KeyReader(raw, where)
    kind = m.string("kind", default="dense")
    if kind == "dense":
        return dict(kind="dense", ff=m.integer("ff"))
    if kind != "moe":
        raise ConfigError(f"{where}: kind {kind!r} is not one of ['dense', 'moe']")
    e = KeyReader(m.raw_value("expert") or {}, where + ".expert")
    r = KeyReader(m.raw_value("router") or {}, where + ".router")
    g = KeyReader(r.raw_value("groups") or {}, where + ".router.groups")
    out = dict(kind="moe", expert=dict(ff=e.integer("ff"), limit=e.number("limit")),
               router=dict(experts=r.integer("experts"), top=r.integer("top"),
                           groups=dict(count=g.integer("count", default=1), keep=g.integer("keep", default=None))))
    ro = out["router"]
    if ro["groups"]["keep"] is None:
        ro["groups"]["keep"] = ro["groups"]["count"]
    n, count, keep = ro["experts"], ro["groups"]["count"], ro["groups"]["keep"]
    if n % count or keep > count or ro["top"] > keep * (n // count):
        raise ConfigError(f"{where}.router: {n} experts in {count} groups, {keep} kept, {ro['top']} chosen do not fit")
    return out


class LagedraConfig:
    architecture = ARCHITECTURE

    def __init__(self, vocab: int, width: int, max_positions: int, eps: float, layers: List[Dict[str, Any]],
                 init_std: Optional[float] = None):
        self.vocab, self.width, self.max_positions, self.eps = vocab, width, max_positions, eps
        self.layers = layers
        self.init_std = init_std
        self._fan_in: Optional[Dict[str, int]] = None

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "LagedraConfig":
        r = KeyReader(raw)
        vocab, width, max_positions = r.integer("vocab"), r.integer("width"), r.integer("max_positions")
        eps = KeyReader(r.raw_value("norm") or {}, "config.json: norm").number("eps")
        raw_layers = r.raw_value("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError(f"config.json: 'layers' must be a non-empty list, found {raw_layers!r}")
        layers: List[Dict[str, Any]] = []
        for i, entry in enumerate(raw_layers):
            where = f"config.json: layers[{i}]"
            e = KeyReader(entry, where)
            kind = e.string("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: type {kind!r} is not one of {list(MIXER_TYPES)}")
            layers.append(dict(type=kind, mixer=_mixer_sizes(kind, e.raw_value("mixer"), where + ".mixer"),
                               mlp=_mlp_sizes(e.raw_value("mlp"), where + ".mlp")))
        blending = [l["mixer"] for l in layers if l["type"] == "attention" and l["mixer"]["v_mix"]]
        if len({(m["kv_heads"], m["vdim"]) for m in blending}) > 1:
            raise ConfigError("config.json: the layers with 'v_mix' blend their values and need equal kv_heads and vdim")
        return cls(vocab, width, max_positions, eps, layers, init_std=raw.get("init_std"))

    def to_dict(self) -> Dict[str, Any]:
        """A config.json that reads back to this configuration."""
        d = dict(architecture=ARCHITECTURE, vocab=self.vocab, width=self.width, max_positions=self.max_positions,
                 norm=dict(eps=self.eps), layers=copy.deepcopy(self.layers))
        if self.init_std is not None:
            d["init_std"] = self.init_std
        return d

    # ---------------------------------------------------------------- description
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("scalar_rmsnorm", dict(size=self.width, eps=self.eps, weight=name))

    def _mixer(self, layer: Dict[str, Any], first_blend: bool) -> PartSpec:
        m = layer["mixer"]
        if layer["type"] == "lightning":
            return PartSpec("lightning_attention", dict(
                hidden_size=self.width, n_heads=m["heads"], dim=m["dim"], v_dim=m["vdim"], decays=tuple(m["decay"]),
                eps=self.eps, q="mix.q", k="mix.k", v="mix.v", g="mix.g", o="mix.o", norm="mix.norm"))
        position = None
        if m["rot"] is not None:
            position = PartSpec("rope_half", dict(dims=m["rot"]["dims"], base=m["rot"]["base"],
                                                  scaling=m["rot"]["scaling"], max_positions=self.max_positions))
        return PartSpec("capped_attention", dict(
            hidden_size=self.width, n_heads=m["heads"], n_kv_heads=m["kv_heads"], dim=m["dim"], v_dim=m["vdim"],
            scale=m["scale"], cap=m["softcap"], window=None if m["mask"] is None else m["mask"]["size"],
            taps=m["conv"], position=position, v_share=V_SHARE if m["v_mix"] else None, v_share_first=first_blend,
            q="mix.q", k="mix.k", v="mix.v", o="mix.o", temp="mix.temp", vmix="mix.vmix"))

    def _feed_forward(self, mlp: Dict[str, Any]) -> PartSpec:
        if mlp["kind"] == "dense":
            return PartSpec("dense_gelu", dict(hidden_size=self.width, intermediate_size=mlp["ff"],
                                               up="mlp.up", down="mlp.down"))
        r = mlp["router"]
        return PartSpec("grouped_moe", dict(
            hidden_size=self.width, intermediate_size=mlp["expert"]["ff"], n_experts=r["experts"], top=r["top"],
            groups=r["groups"]["count"], keep=r["groups"]["keep"], limit=mlp["expert"]["limit"],
            router="mlp.router", expert="mlp.e{}"))

    def model_spec(self) -> ModelSpec:
        blocks, seen_blend = [], False
        for i, layer in enumerate(self.layers):
            blends = layer["type"] == "attention" and layer["mixer"]["v_mix"]
            norms = {"mixer": self._norm("norm1")}
            ffn = None
            if layer["mlp"] is not None:
                ffn = self._feed_forward(layer["mlp"])
                norms["feed_forward"] = self._norm("norm2")
            blocks.append(BlockSpec(kind="parallel", prefix=f"l{i}.", mixer=self._mixer(layer, blends and not seen_blend),
                                    feed_forward=ffn, norms=norms,
                                    combiner=PartSpec("depth_average", dict(inputs=i + 2, weight="dwa"))))
            seen_blend = seen_blend or blends
        embedding = PartSpec("token_position_embedding", dict(name="embed", positions="pos", vocab_size=self.vocab,
                                                              hidden_size=self.width, max_positions=self.max_positions))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, embedding=embedding, head_name="head",
                         final_norm=self._norm("final.norm"), blocks=tuple(blocks),
                         schedule=straight_schedule(len(blocks)), max_positions=self.max_positions, stop_tokens=())

    def ignored_tensors(self) -> Tuple[str, ...]:
        """What a file may hold without the configuration having a use for it: the norm in front of a
        feed-forward that a layer does not have, the blend of a layer that does not blend its values, the taps
        of a layer without a convolution."""
        names = []
        for i, layer in enumerate(self.layers):
            if layer["mlp"] is None:
                names.append(f"l{i}.norm2")
            if layer["type"] == "attention":
                if not layer["mixer"]["v_mix"]:
                    names.append(f"l{i}.mix.vmix")
                if layer["mixer"]["conv"] is None:
                    names += [f"l{i}.mix.{k}.conv" for k in ("q", "k", "v")]
        return tuple(names)

    def random_init_std(self, tensor_name: str) -> float:
        """Standard deviation for random weights: `init_std` where the configuration gives one, else
        1/sqrt(inputs) for matrices, 1 for the two tables' rows and 0.3 for everything else."""
        if self.init_std is not None:
            return float(self.init_std)
        if self._fan_in is None:
            from ..engine.model import expected_tensors
            self._fan_in = {n: (ts.shape[1] if len(ts.shape) == 2 else 0)
                            for n, ts in expected_tensors(self.model_spec()).items()}
        if tensor_name in ("embed", "pos"):
            return 1.0
        if tensor_name.endswith(".conv"):
            return 0.5
        fan = self._fan_in.get(tensor_name, 0)
        return 1.0 / math.sqrt(fan) if fan else 0.3
