"""Small Tabezen configurations that differ in every size and option, and a writer of model folders
with random weights whose norm gains, biases and activation numbers are not the trivial ones."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def latent(heads, dim, rot_dim, vdim, rank, scale, base=10000.0, dims=None, scaling=None):
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, scale=scale,
                rot=dict(base=base, dims=rot_dim if dims is None else dims, scaling=scaling))


# three norm groups; a recurrent layer first; an attention layer without feed-forward whose tensors
# a later layer borrows; no frequency scaling
TZ_A = dict(architecture="Tabezen", vocab=300, width=96, norm=dict(eps=1e-5, groups=3), layers=[
    dict(type="mingru", mixer=dict(width=80), mlp=dict(kind="dense", ff=112)),
    dict(type="latent_attention", mixer=latent(3, 16, 8, 24, 40, 0.3, base=1000.0), mlp=None),
    dict(type="latent_attention", mixer=latent(3, 16, 8, 24, 40, 0.3, base=1000.0), mlp=None, weights_of=1),
])

# one norm group; five heads; fewer rotated values than the rotated part holds; a stretched frequency
# ladder; a sharp softmax (scale 1.5: single keys decide); a borrowed recurrent layer; two attention
# layers of different sizes, one with a latent of more than 256 values
TZ_B = dict(architecture="Tabezen", vocab=512, width=128, norm=dict(eps=1e-6, groups=1), layers=[
    dict(type="latent_attention",
         mixer=latent(5, 24, 16, 8, 72, 1.5, base=500.0, dims=12, scaling=dict(factor=4.0, original=64, fast=8.0, slow=2.0)),
         mlp=dict(kind="dense", ff=200)),
    dict(type="mingru", mixer=dict(width=300), mlp=dict(kind="dense", ff=64)),
    dict(type="mingru", mixer=dict(width=300), mlp=dict(kind="dense", ff=64), weights_of=1),
    dict(type="latent_attention", mixer=latent(2, 8, 4, 40, 264, 0.7, base=50000.0), mlp=dict(kind="dense", ff=96)),
])

# four groups, a single head, one layer of each kind, the recurrent one without feed-forward
TZ_C = dict(architecture="Tabezen", vocab=97, width=64, norm=dict(eps=1e-4, groups=4), layers=[
    dict(type="latent_attention",
         mixer=latent(1, 32, 16, 16, 24, 0.2, base=20.0, scaling=dict(factor=16.0, original=32, fast=4.0, slow=1.0)),
         mlp=dict(kind="dense", ff=48)),
    dict(type="mingru", mixer=dict(width=40), mlp=None),
])

TZ = {"A": TZ_A, "B": TZ_B, "C": TZ_C}


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)


def write_tabezen(folder: str, raw: dict, seed: int = 0, sharpen: float = 1.0) -> str:
    """config.json and model.safetensors (bfloat16).  Matrices N(0, 1/inputs), norm gains around one,
    biases and the activation's numbers of order one; `sharpen` scales the query matrices."""
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    from minfer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    expected = expected_tensors(config_from_dict(raw).model_spec())
    rng = np.random.default_rng(seed)
    made = {}
    for name, ts in expected.items():
        shape = tuple(ts.shape)
        if "norm" in name:
            a = 1.0 + 0.3 * rng.standard_normal(shape)
        elif name.endswith(".act"):
            a = rng.standard_normal(shape)
        elif len(shape) == 1:
            a = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[1])
            if name.endswith("mix.q"):
                a = a * sharpen
        made[name] = _bf16(a)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(n, tuple(t.shape), torch.bfloat16) for n, t in made.items()], lambda n: made[n])
    return folder


def random_config(rng) -> dict:
    """A configuration drawn at random: widths and vocabularies that are multiples of nothing useful,
    one to five layers of either kind in any order, borrowed tensors, layers without feed-forward, odd
    head sizes, ranks and value widths, fewer rotated values than the rotated part holds, plain and
    stretched frequency ladders."""
    width = int(rng.choice([48, 64, 100, 128, 136, 192, 256, 320]))
    groups = int(rng.choice([g for g in (1, 2, 4, 5, 8, 3) if width % g == 0]))
    layers = []
    for _ in range(int(rng.integers(1, 6))):
        if layers and rng.random() < 0.25:
            j = int(rng.integers(0, len(layers)))
            if "weights_of" not in layers[j]:
                layers.append(dict(layers[j], weights_of=j))
                continue
        mlp = None if rng.random() < 0.2 else dict(kind="dense", ff=int(rng.choice([40, 64, 100, 256, 384, 777])))
        if rng.random() < 0.45:
            layers.append(dict(type="mingru", mixer=dict(width=int(rng.choice([24, 64, 100, 256, 384, 513]))), mlp=mlp))
            continue
        rot_dim = int(rng.choice([2, 4, 8, 16, 32, 64, 6]))
        dims = int(rng.choice([d for d in (2, 4, 6, 8, 16, 32, 64) if d <= rot_dim]))
        scaling = None
        if rng.random() < 0.7:
            scaling = dict(factor=float(rng.choice([2.0, 8.0, 32.0])), original=int(rng.choice([16, 128, 1024, 4096])),
                           fast=float(rng.choice([8.0, 32.0])), slow=float(rng.choice([1.0, 2.0])))
        layers.append(dict(type="latent_attention", mlp=mlp, mixer=latent(
            int(rng.choice([1, 2, 3, 4, 6, 8, 16])), int(rng.choice([8, 16, 24, 32, 64, 5])), rot_dim,
            int(rng.choice([8, 16, 32, 48, 64, 7])), int(rng.choice([16, 32, 64, 96, 128, 256, 30])),
            float(rng.choice([0.05, 0.125, 0.3])), base=float(rng.choice([100.0, 10000.0, 500000.0])), dims=dims,
            scaling=scaling)))
    return dict(architecture="Tabezen", vocab=int(rng.choice([64, 300, 512, 1000])), width=width,
                norm=dict(eps=float(rng.choice([1e-6, 1e-5])), groups=groups), layers=layers)
