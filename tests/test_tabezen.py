"""Tabezen without a GPU: the configuration, the plain implementation's own mechanisms against
hand-made cases, and the real engine, cache and generation loop driven through the plain stand-ins
for the kernels against the plain implementation."""
import math

import numpy as np
import pytest
import torch

import plain_ops
import plain_tabezen as pt
from replays import batch_steps, chunk_steps, requests_for, run_steps, tail_steps, whole_steps
from tabezen_tiny import TZ, TZ_A, TZ_B, write_tabezen


# ------------------------------------------------------------------ configuration
def test_configuration_reads_writes_and_describes():
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    cfg = config_from_dict(TZ_B)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.model_spec()
    assert len(spec.blocks) == 3 and [e.block for e in spec.schedule] == [0, 1, 1, 2]
    assert [e.cache for e in spec.schedule] == [0, 1, 2, 3]
    names = expected_tensors(spec)
    assert names["l0.mix.dkv"].shape == (72 + 16, 128) and names["l0.mix.g"].shape == (5, 128)
    assert names["l3.mix.uv"].shape == (2 * 40, 264) and names["l1.mix.z.b"].shape == (300,)
    assert not any(n.startswith("l2.") for n in names) and "embed.norm" in names and "final.norm" in names


@pytest.mark.parametrize("change, word", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2]["mixer"].update(width=301), "borrows"),
    (lambda c: c["norm"].update(groups=5), "groups"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "dims"),
    (lambda c: c.pop("vocab"), "vocab"),
])
def test_configuration_rejections_name_the_key(change, word):
    import copy
    from minfer_amd import ConfigError, config_from_dict
    raw = copy.deepcopy(TZ_B)
    change(raw)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(raw)


# ------------------------------------------------------------------ the plain mechanisms by hand
def test_plain_group_norm_by_hand():
    x = np.array([[3.0, 4.0, 0.0, 2.0]])
    y = pt.group_rms_norm(x, np.array([1.0, 2.0, 1.0, 0.5]), 0.0, 2)
    assert np.allclose(y, [[3 / math.sqrt(12.5), 8 / math.sqrt(12.5), 0.0, 0.5 * 2 / math.sqrt(2.0)]])
    assert np.allclose(pt.group_rms_norm(x, np.ones(4), 0.0, 1), x / math.sqrt(29 / 4))


def test_plain_xielu_by_hand():
    p, q = 0.3, -0.2
    sp = lambda v: math.log1p(math.exp(v))
    z = np.array([2.0, -1.0, 0.0])
    want = [sp(p) * 4 + 1.0, (0.5 + sp(q)) * (math.exp(-1) - 1 + 1) - 0.5, 0.0]
    assert np.allclose(pt.xielu(z, p, q), want)


def test_plain_frequency_ladder_by_hand():
    f, mag = pt.yarn_frequencies(8, 100.0, None)
    assert np.allclose(f, [1.0, 100 ** -0.25, 0.1, 100 ** -0.75]) and mag == 1.0
    sc = dict(factor=4.0, original=64, fast=8.0, slow=2.0)
    f2, mag2 = pt.yarn_frequencies(8, 100.0, sc)
    pair = lambda t: 8 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(pair(8.0)), 0), min(math.ceil(pair(2.0)), 7)
    ramp = [min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001))) for i in range(4)]
    assert np.allclose(f2, [fi / 4 * r + fi * (1 - r) for fi, r in zip(f, ramp)])
    assert mag2 == pytest.approx(0.1 * math.log(4.0) + 1.0)
    # pairs (2i, 2i+1), values behind `dims` untouched, position 0 only scaled
    x = np.arange(12, dtype=np.float64).reshape(2, 6)
    y = pt.rotate_interleaved(x, [0, 3], 4, 100.0, None)
    assert np.allclose(y[0], x[0]) and np.allclose(y[1, 4:], x[1, 4:])
    assert np.allclose(y[1, :2], [6 * math.cos(3) - 7 * math.sin(3), 7 * math.cos(3) + 6 * math.sin(3)])


def test_plain_mingru_by_hand_and_carried_state():
    rng = np.random.default_rng(0)
    w = {"z": rng.standard_normal((3, 4)), "z.b": rng.standard_normal(3), "x": rng.standard_normal((3, 4)),
         "x.b": rng.standard_normal(3), "g": rng.standard_normal((3, 4)), "o": rng.standard_normal((4, 3))}
    h = rng.standard_normal((6, 4))
    out, s = pt.mingru(h, w)
    z0 = pt.sigmoid(h[0] @ w["z"].T + w["z.b"])
    u0 = h[0] @ w["x"].T + w["x.b"]
    c0 = np.where(u0 >= 0, u0 + 0.5, pt.sigmoid(u0))
    assert np.allclose(out[0], (z0 * c0 * pt.silu(h[0] @ w["g"].T)) @ w["o"].T)
    a, sa = pt.mingru(h[:4], w)
    b, sb = pt.mingru(h[4:], w, sa)
    assert np.allclose(np.concatenate([a, b]), out) and np.allclose(sb, s)


def test_plain_latent_attention_equals_explicit_keys_and_values():
    """One token's result put together from explicit per-head keys and values."""
    rng = np.random.default_rng(1)
    m = dict(heads=2, dim=3, rot_dim=4, vdim=5, kv_rank=6, scale=0.4, rot=dict(base=50.0, dims=2, scaling=None))
    W = 7
    w = {"q": rng.standard_normal((2 * 7, W)), "dkv": rng.standard_normal((10, W)), "dkv.norm": rng.standard_normal(6),
         "uk": rng.standard_normal((6, 6)), "uv": rng.standard_normal((10, 6)), "g": rng.standard_normal((2, W)),
         "o": rng.standard_normal((W, 10))}
    h = rng.standard_normal((5, W))
    out = pt.latent_attention(h, w, m, 1e-6)
    t = 4
    lat = h @ w["dkv"].T
    c = lat[:, :6] / np.sqrt((lat[:, :6] ** 2).mean(-1, keepdims=True) + 1e-6) * w["dkv.norm"]
    heads = []
    for hd in range(2):
        q = h[t] @ w["q"][hd * 7:(hd + 1) * 7].T
        qr = pt.rotate_interleaved(q[None, 3:], [t], 2, 50.0, None)[0]
        s = []
        for j in range(t + 1):
            kr = pt.rotate_interleaved(lat[j:j + 1, 6:], [j], 2, 50.0, None)[0]
            s.append((q[:3] @ (w["uk"][hd * 3:(hd + 1) * 3] @ c[j]) + qr @ kr) * 0.4)
        p = np.exp(np.array(s) - max(s))
        p /= p.sum()
        v = sum(p[j] * (w["uv"][hd * 5:(hd + 1) * 5] @ c[j]) for j in range(t + 1))
        heads.append(v * pt.sigmoid(h[t] @ w["g"][hd]))
    assert np.allclose(out[t], np.concatenate(heads) @ w["o"].T)


# ------------------------------------------------------------------ the engine through the stand-ins
def _rel(rows, ref):
    worst = 0.0
    for (rid, p), got in rows.items():
        want = ref[rid][p]
        worst = max(worst, float(np.abs(got - want).max() / max(1e-9, want.std())))
    return worst


@pytest.mark.parametrize("name", list(TZ))
def test_engine_on_stand_ins_agrees_with_plain(tmp_path, monkeypatch, name):
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, load_model
    folder = write_tabezen(str(tmp_path / name), TZ[name], seed=5)
    plain = pt.PlainTabezen.from_folder(folder)
    reqs = requests_for(TZ[name]["vocab"], (1, 7, 70, 33, 150), seed=2)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 12)
    ids = list(reqs)
    for what, steps in (("whole", whole_steps(reqs)), ("one by one", tail_steps(reqs, tail=9)),
                        ("batches", batch_steps(reqs, [ids[:3], ids[3:]])),
                        ("portions", chunk_steps(reqs, [ids[:2], ids[2:]], sizes=(2, 50, 64, 1, 17)))):
        assert _rel(run_steps(eng, steps), ref) < 1e-4, what
    assert not eng.cache.live_slots()


def test_greedy_generation_on_stand_ins(tmp_path, monkeypatch):
    """`generate` with its scheduler, slots and decode sessions, tokens against the plain model."""
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, generate, load_model
    from minfer_amd.sampling import SamplingParams
    folder = write_tabezen(str(tmp_path / "gen"), TZ_A, seed=8)
    plain = pt.PlainTabezen.from_folder(folder)
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 6, max_seqs=2)
    prompts = [[5, 9, 200, 7], [11], [250, 3, 3, 3, 8, 1, 44]]
    res = generate(eng, prompts, SamplingParams(temp=0.0, repeat_penalty=1.0), max_new=5, stop_tokens=[])
    for p, toks in zip(prompts, res.tokens):
        seq = list(p)
        for t in toks:
            assert t == pt.greedy(plain.forward(seq)[-1])
            seq.append(t)
    assert not eng.cache.live_slots()
