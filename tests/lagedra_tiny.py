"""Small Lagedra configurations that differ in every size and option, a writer of model folders with
random weights whose gains (0.6 to 1.4), sum weights, temperatures and blends are not the trivial ones, and
configurations drawn at random."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, scale, window=None, conv=None, softcap=None, rot_dims=None, base=10000.0,
              scaling=None, v_mix=False):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, v_mix=v_mix)
    if window is not None:
        m["mask"] = dict(size=window)
    if conv is not None:
        m["conv"] = conv
    if softcap is not None:
        m["softcap"] = softcap
    if rot_dims is not None:
        m["rot"] = dict(base=base, dims=rot_dims, scaling=scaling)
    return dict(type="attention", mixer=m)


def lightning(heads, dim, vdim, decay):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)))


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, count, keep, ff, limit):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit),
                router=dict(experts=experts, top=top, groups=dict(count=count, keep=keep)))


# attention first; values blended over two attention layers with a lightning layer without feed-forward
# between them; rotation over part of a head without and over the whole head with a stretched ladder;
# windows of 17 and 70; four and two taps; a capped and an uncapped layer; six experts in three groups
LG_A = dict(architecture="Lagedra", vocab=300, width=96, max_positions=512, norm=dict(eps=1e-5), layers=[
    dict(attention(6, 3, 24, 40, 0.25, window=17, conv=4, softcap=8.0, rot_dims=16, base=1000.0, v_mix=True), mlp=dense(112)),
    dict(lightning(3, 20, 12, (0.9, 0.5, 1.0)), mlp=None),
    dict(attention(3, 3, 24, 40, 0.4, window=70, conv=2, rot_dims=24, base=500.0,
                   scaling=dict(factor=4.0, original=64, fast=8.0, slow=2.0), v_mix=True),
         mlp=moe(6, 3, 3, 2, 40, 1.5)),
])

# a single lightning head wider in its values than in its keys with one expert of four; attention without
# convolution, rotation, window, cap or blending; nine query heads on one kv head (more than a workgroup
# takes at once), a window of five and a convolution of one tap
LG_B = dict(architecture="Lagedra", vocab=512, width=128, max_positions=400, norm=dict(eps=1e-6), layers=[
    dict(lightning(1, 40, 72, (0.97,)), mlp=moe(4, 1, 1, 1, 56, 0.7)),
    dict(attention(4, 4, 16, 16, 0.3), mlp=dense(200)),
    dict(attention(9, 1, 8, 24, 0.6, window=5, conv=1, softcap=2.0, rot_dims=4, base=50.0,
                   scaling=dict(factor=16.0, original=32, fast=4.0, slow=1.0)), mlp=None),
    dict(lightning(2, 136, 16, (0.2, 0.999)), mlp=dense(64)),
])

# sizes that are multiples of nothing: keys of 12 and 5, values of 5 and 7, a window of one (a token sees
# itself only), eight experts all in play, three layers that blend
LG_C = dict(architecture="Lagedra", vocab=97, width=64, max_positions=300, norm=dict(eps=1e-4), layers=[
    dict(lightning(3, 5, 7, (0.8, 0.6, 0.95)), mlp=dense(48)),
    dict(attention(2, 1, 12, 5, 0.5, window=1, conv=3, softcap=30.0, rot_dims=2, base=20.0, v_mix=True), mlp=moe(8, 8, 4, 4, 24, 3.0)),
    dict(attention(4, 1, 10, 5, 0.35, window=64, conv=5, rot_dims=10, base=10000.0, v_mix=True), mlp=dense(80)),
    dict(attention(1, 1, 16, 5, 0.3, window=65, conv=2, softcap=5.0, v_mix=True), mlp=None),
])

LG = {"A": LG_A, "B": LG_B, "C": LG_C}


def _bf16(a) -> torch.Tensor:
    return torch.tensor(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)       # (a single number keeps its empty shape)


def write_lagedra(folder: str, raw: dict, seed: int = 0, sharpen: float = 1.0) -> str:
    """config.json and model.safetensors (bfloat16).  Matrices N(0, 1/inputs); gains, temperatures and the
    norm over the lightning heads around one; the depth sums' weights around an even share with the
    newest result favoured; blends between 0.2 and 0.6; `sharpen` scales the attention's query matrices."""
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
        if name.endswith(".dwa"):
            a = 0.3 * rng.standard_normal(shape) / shape[0]
            a[-1] += 1.0
        elif name.endswith(".vmix"):
            a = rng.uniform(0.2, 0.6, shape)
        elif "norm" in name or name.endswith(".temp"):
            a = rng.uniform(0.6, 1.4, shape)
        elif name.endswith(".conv"):
            a = rng.standard_normal(shape) / np.sqrt(shape[1])
        elif name in ("embed", "pos"):
            a = rng.standard_normal(shape) * (1.0 if name == "embed" else 0.5)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[1])
            if name.endswith("mix.q") and (len(shape) == 2) and any(
                    l["type"] == "attention" for i, l in enumerate(raw["layers"]) if name.startswith(f"l{i}.")):
                a = a * sharpen
        made[name] = _bf16(a)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(n, tuple(t.shape), torch.bfloat16) for n, t in made.items()], lambda n: made[n])
    return folder


def random_config(rng) -> dict:
    """A configuration drawn at random: one to five layers of either kind in any order, with and without
    feed-forward, dense or routed, odd head sizes and counts, windows from one to beyond the prompts,
    convolutions of one to six taps or none, partial and whole rotations with and without a stretched
    ladder, capped or not, blended or not."""
    width = int(rng.choice([48, 64, 100, 128, 136, 192, 256]))
    layers = []
    blend_shape = (int(rng.choice([1, 2, 3])), int(rng.choice([8, 16, 20, 48, 7])))
    for _ in range(int(rng.integers(1, 6))):
        r = rng.random()
        if r < 0.2:
            mlp = None
        elif r < 0.6:
            mlp = dense(int(rng.choice([40, 64, 100, 256, 333])))
        else:
            count = int(rng.choice([1, 2, 4]))
            per = int(rng.choice([1, 2, 3]))
            keep = int(rng.integers(1, count + 1))
            mlp = moe(count * per, int(rng.integers(1, keep * per + 1)), count, keep, int(rng.choice([16, 40, 64, 72])),
                      float(rng.choice([0.5, 2.0, 7.0])))
        if rng.random() < 0.4:
            heads = int(rng.choice([1, 2, 3, 5]))
            layers.append(dict(lightning(heads, int(rng.choice([4, 16, 24, 64, 96, 130])), int(rng.choice([8, 16, 40, 64, 100])),
                                         [float(d) for d in rng.uniform(0.3, 1.0, heads)]), mlp=mlp))
            continue
        blends = rng.random() < 0.6
        kv = blend_shape[0] if blends else int(rng.choice([1, 2, 4]))
        vdim = blend_shape[1] if blends else int(rng.choice([8, 16, 24, 64, 5]))
        dim = int(rng.choice([8, 16, 24, 32, 64, 96, 6]))
        rot = None if rng.random() < 0.15 else int(rng.choice([d for d in (2, 4, 6, 8, 16, 32, 64, 96) if d <= dim]))
        scaling = None
        if rot is not None and rng.random() < 0.6:
            scaling = dict(factor=float(rng.choice([2.0, 8.0, 32.0])), original=int(rng.choice([16, 128, 1024])),
                           fast=float(rng.choice([8.0, 32.0])), slow=float(rng.choice([1.0, 2.0])))
        layers.append(dict(attention(
            kv * int(rng.choice([1, 2, 3, 10])), kv, dim, vdim, float(rng.choice([0.05, 0.125, 0.3])),
            window=None if rng.random() < 0.2 else int(rng.choice([1, 2, 31, 64, 65, 100, 1000])),
            conv=None if rng.random() < 0.2 else int(rng.integers(1, 7)),
            softcap=None if rng.random() < 0.3 else float(rng.choice([1.0, 10.0, 50.0])),
            rot_dims=rot, base=float(rng.choice([100.0, 10000.0, 500000.0])), scaling=scaling, v_mix=blends), mlp=mlp))
    return dict(architecture="Lagedra", vocab=int(rng.choice([64, 300, 512, 1000])), width=width, max_positions=512,
                norm=dict(eps=float(rng.choice([1e-6, 1e-5]))), layers=layers)
