"""Tabezen: a decoder whose layers mix tokens either with a minGRU recurrence or with attention
over a shared low-rank latent, whose branches read the residual stream itself and are normed on
their way back into it, and whose norm is an RMS norm taken in groups.

config.json: `architecture` = "Tabezen"; `vocab`, `width`; `norm` = {eps, groups}; `layers`, a list
of {type: "mingru" | "latent_attention", mixer: {...sizes...}, mlp: {kind: "dense", ff} or null,
weights_of: j (optional: the layer has no tensors of its own and runs layer j's, with a cache or
state of its own)}.  Mixer sizes: mingru {width}; latent_attention {heads, dim, rot_dim, vdim,
kv_rank, scale, rot: {base, dims, scaling: {factor, original, fast, slow} or null}}.
Tensors: embed, embed.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""
from __future__ import annotations

import copy
import math
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError, KeyReader
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE = "Tabezen"
MIXER_TYPES = ("mingru", "latent_attention")
# the design names no bound on positions; the rotation tables grow on demand up to this
MAX_POSITIONS = 1 << 20


def _mixer_sizes(kind: str, raw: Any, where: str) -> Dict[str, Any]:
    r = KeyReader(raw, where)
    if kind == "mingru":
        return dict(width=r.integer("width"))
    out = dict(heads=r.integer("heads"), dim=r.integer("dim"), rot_dim=r.integer("rot_dim"),
               vdim=r.integer("vdim"), kv_rank=r.integer("kv_rank"), scale=r.number("scale"))
    rot = KeyReader(r.raw_value("rot") or {}, where + ".rot")
    dims = rot.integer("dims", default=out["rot_dim"])
    if dims % 2 or dims > out["rot_dim"]:
        raise ConfigError(f"{where}.rot: 'dims' must be even and at most rot_dim {out['rot_dim']}, found {dims}")
    scaling = rot.raw_value("scaling")
    if scaling is not None:
        s = KeyReader(scaling, where + ".rot.scaling")
        scaling = dict(factor=s.number("factor"), original=s.number("original"), fast=s.number("fast"),
                       slow=s.number("slow"))
    out["rot"] = dict(base=rot.number("base"), dims=dims, scaling=scaling)
    return out


class TabezenConfig:
    architecture = ARCHITECTURE

    def __init__(self, vocab: int, width: int, eps: float, groups: int, layers: List[Dict[str, Any]],
                 init_std: Optional[float] = None):
        self.vocab, self.width, self.eps, self.groups = vocab, width, eps, groups
        self.layers = layers
        self.init_std = init_std
        self._fan_in: Optional[Dict[str, int]] = None

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "TabezenConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab"), r.integer("width")
        norm = KeyReader(r.raw_value("norm") or {}, "config.json: norm")
        eps, groups = norm.number("eps"), norm.integer("groups", default=1)
        if width % groups:
            raise ConfigError(f"config.json: width {width} does not split into norm.groups {groups} equal parts")
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
            mixer = _mixer_sizes(kind, e.raw_value("mixer"), where + ".mixer")
            mlp = e.raw_value("mlp")
            if mlp is not None:
                m = KeyReader(mlp, where + ".mlp")
                mlp_kind = m.string("kind", default="dense")
                if mlp_kind != "dense":
                    raise ConfigError(f"{where}.mlp: kind {mlp_kind!r} is not supported; only 'dense'")
                mlp = dict(kind="dense", ff=m.integer("ff"))
            owner = e.integer("weights_of", default=None, minimum=0)
            layers.append(dict(type=kind, mixer=mixer, mlp=mlp, weights_of=owner))
        for i, layer in enumerate(layers):
            j = layer["weights_of"]
            if j is None:
                continue
            if j >= len(layers) or j == i or layers[j]["weights_of"] is not None:
                raise ConfigError(f"config.json: layers[{i}].weights_of {j} must name another layer that has tensors of its own")
            if any(layers[j][k] != layer[k] for k in ("type", "mixer", "mlp")):
                raise ConfigError(f"config.json: layers[{i}] borrows layer {j}'s tensors but differs from it")
        return cls(vocab, width, eps, groups, layers, init_std=raw.get("init_std"))

    def to_dict(self) -> Dict[str, Any]:
        """A config.json that reads back to this configuration."""
        layers = []
        for layer in self.layers:
            e = dict(type=layer["type"], mixer=copy.deepcopy(layer["mixer"]), mlp=copy.deepcopy(layer["mlp"]))
            if layer["weights_of"] is not None:
                e["weights_of"] = layer["weights_of"]
            layers.append(e)
        d = dict(architecture=ARCHITECTURE, vocab=self.vocab, width=self.width,
                 norm=dict(eps=self.eps, groups=self.groups), layers=layers)
        if self.init_std is not None:
            d["init_std"] = self.init_std
        return d

    # ---------------------------------------------------------------- description
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("group_rmsnorm", dict(size=self.width, eps=self.eps, groups=self.groups, weight=name))

    def _mixer(self, layer: Dict[str, Any]) -> PartSpec:
        m = layer["mixer"]
        if layer["type"] == "mingru":
            return PartSpec("mingru", dict(hidden_size=self.width, width=m["width"],
                                           z="mix.z", x="mix.x", g="mix.g", o="mix.o"))
        rot = m["rot"]
        position = PartSpec("rope_pairs", dict(dims=rot["dims"], base=rot["base"], scaling=rot["scaling"],
                                               max_positions=MAX_POSITIONS))
        return PartSpec("latent_attention", dict(
            hidden_size=self.width, n_heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], v_dim=m["vdim"],
            rank=m["kv_rank"], scale=m["scale"], eps=self.eps, window=None, position=position,
            q="mix.q", dkv="mix.dkv", dkv_norm="mix.dkv.norm", uk="mix.uk", uv="mix.uv", gate="mix.g", o="mix.o"))

    def model_spec(self) -> ModelSpec:
        """Layers with tensors of their own become blocks; the run order lists every layer, a
        borrowing layer as one more run of its owner's block with a cache entry of its own."""
        blocks, index_of = [], {}
        for i, layer in enumerate(self.layers):
            if layer["weights_of"] is not None:
                continue
            ffn, norms = None, {"mixer_out": self._norm("norm1")}
            if layer["mlp"] is not None:
                ffn = PartSpec("dense_xielu", dict(hidden_size=self.width, intermediate_size=layer["mlp"]["ff"],
                                                   up="mlp.up", down="mlp.down", act="mlp.act"))
                norms["feed_forward_out"] = self._norm("norm2")
            index_of[i] = len(blocks)
            blocks.append(BlockSpec(kind="branch_norm", prefix=f"l{i}.", mixer=self._mixer(layer), feed_forward=ffn,
                                    norms=norms))
        schedule = tuple(RunEntry(block=index_of[i if layer["weights_of"] is None else layer["weights_of"]], cache=i)
                         for i, layer in enumerate(self.layers))
        embedding = PartSpec("normed_token_embedding", dict(name="embed", vocab_size=self.vocab, hidden_size=self.width,
                                                            norm=self._norm("embed.norm")))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, embedding=embedding, head_name="head",
                         final_norm=self._norm("final.norm"), blocks=tuple(blocks), schedule=schedule,
                         max_positions=MAX_POSITIONS, stop_tokens=())

    def ignored_tensors(self) -> Tuple[str, ...]:
        return ()

    def random_init_std(self, tensor_name: str) -> float:
        """Standard deviation for random weights: `init_std` where the configuration gives one, else
        1/sqrt(inputs) for matrices, 0.1 for biases and 0.5 for the activation's two numbers."""
        if self.init_std is not None:
            return float(self.init_std)
        if self._fan_in is None:
            from ..engine.model import expected_tensors
            self._fan_in = {n: (ts.shape[1] if len(ts.shape) == 2 else 0)
                            for n, ts in expected_tensors(self.model_spec()).items()}
        fan = self._fan_in.get(tensor_name, 0)
        if tensor_name.endswith(".act"):
            return 0.5
        if tensor_name == "embed":
            return 1.0
        return 1.0 / math.sqrt(fan) if fan else 0.1
