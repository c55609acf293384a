"""Lagedra without a GPU: the configuration, the plain implementation's own mechanisms against
hand-made cases, and the real engine, cache and generation loop driven through the plain stand-ins
for the kernels against the plain implementation."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_lagedra as pl
import plain_ops
from lagedra_tiny import LG, LG_A, LG_B, LG_C, random_config, write_lagedra
from replays import batch_steps, chunk_steps, requests_for, run_steps, tail_steps, whole_steps


# ------------------------------------------------------------------ configuration
def test_configuration_reads_writes_and_describes():
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    cfg = config_from_dict(LG_A)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.model_spec()
    assert [b.kind for b in spec.blocks] == ["parallel"] * 3 and [e.cache for e in spec.schedule] == [0, 1, 2]
    assert [b.combiner.params["inputs"] for b in spec.blocks] == [2, 3, 4]
    assert spec.blocks[0].mixer.params["v_share_first"] and not spec.blocks[2].mixer.params["v_share_first"]
    names = expected_tensors(spec)
    assert names["l0.mix.q"].shape == (6 * 24, 96) and names["l0.mix.v"].shape == (3 * 40, 96)
    assert names["l0.mix.k.conv"].shape == (3 * 24, 4) and names["l2.mix.v.conv"].shape == (3 * 40, 2)
    assert names["l0.norm1"].shape == () and names["l2.mix.vmix"].shape == () and names["l2.dwa"].shape == (4,)
    assert names["l1.mix.norm"].shape == (36,) and "l1.norm2" not in names and "l1.mlp.up" not in names
    assert names["l2.mlp.router"].shape == (6, 96) and names["l2.mlp.e5.down"].shape == (96, 40)
    assert names["pos"].shape == (512, 96) and names["final.norm"].shape == ()
    other = expected_tensors(config_from_dict(LG_B).model_spec())
    assert "l1.mix.q.conv" not in other and "l1.mix.vmix" not in other and other["l2.mix.q.conv"].shape == (72, 1)


@pytest.mark.parametrize("change, word", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5, 0.5]), "decay"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=26), "dims"),
    (lambda c: c["layers"][2]["mlp"]["router"].update(top=5), "router"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=8), "v_mix"),
    (lambda c: c.pop("max_positions"), "max_positions"),
])
def test_configuration_rejections_name_the_key(change, word):
    from minfer_amd import ConfigError, config_from_dict
    raw = copy.deepcopy(LG_A)
    change(raw)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(raw)


# ------------------------------------------------------------------ the plain mechanisms by hand
def test_plain_norm_gelu_and_expert_by_hand():
    x = np.array([[3.0, 4.0, 0.0, 0.0]])
    assert np.allclose(pl.scalar_rms_norm(x, 0.5, 0.0), 0.5 * x / math.sqrt(25 / 4))
    assert np.allclose(pl.gelu_tanh(np.array([0.0, 1.0])), [0.0, 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715))])
    h = np.array([1.0, -2.0])
    gate, up, down = np.array([[3.0, 0.0], [0.0, 1.0]]), np.array([[-4.0, 0.0], [1.0, 1.0]]), np.eye(2)
    g = np.array([2.0, -2.0])                    # min(3, 2), -2
    u = np.array([-2.0, -1.0])                   # clamp(-4), 1 - 2
    assert np.allclose(pl.expert(h, gate, up, down, 2.0), g / (1 + np.exp(-1.702 * g)) * (u + 1))


def test_plain_router_by_hand():
    # scores rise with the logits; groups of two neighbours: (0,1) (2,3) (4,5); the best group holds expert 5,
    # the second best expert 2; expert 1 is the third best expert but its group is not kept
    z = np.log(np.array([0.05, 0.2, 0.25, 0.02, 0.03, 0.45]))
    chosen, w = pl.route(z, 3, 3, 2)
    assert list(chosen) == [5, 2, 4] and np.allclose(w, np.array([0.45, 0.25, 0.03]) / 0.73)
    chosen, w = pl.route(z, 2, 1, 1)
    assert list(chosen) == [5, 2] and np.allclose(w.sum(), 1.0)


def test_plain_convolution_by_hand_and_carried():
    u = np.arange(10, dtype=np.float64).reshape(5, 2) + 1
    w = np.array([[1.0, 10.0, 100.0], [0.0, 0.0, 2.0]])
    y, last = pl.causal_conv(u, w)
    assert np.allclose(y[0], [100 * 1, 2 * 2]) and np.allclose(y[1], [10 * 1 + 100 * 3, 2 * 4])
    assert np.allclose(y[4], [1 * 5 + 10 * 7 + 100 * 9, 2 * 10]) and np.allclose(last, u[3:])
    a, sa = pl.causal_conv(u[:1], w)
    b, sb = pl.causal_conv(u[1:], w, sa)
    assert np.allclose(np.concatenate([a, b]), y) and np.allclose(sb, last)


def test_plain_half_rotation_by_hand():
    f, mag = pl.yarn_frequencies(8, 100.0, None)
    assert np.allclose(f, [1.0, 100 ** -0.25, 0.1, 100 ** -0.75]) and mag == 1.0
    sc = dict(factor=4.0, original=64, fast=8.0, slow=2.0)
    f2, mag2 = pl.yarn_frequencies(8, 100.0, sc)
    index = lambda t: 8 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(index(8.0)), 0), min(math.ceil(index(2.0)), 7)
    ramp = [min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001))) for i in range(4)]
    assert np.allclose(f2, [fi / 4 * r + fi * (1 - r) for fi, r in zip(f, ramp)])
    assert mag2 == pytest.approx(0.1 * math.log(4.0) + 1.0)
    x = np.arange(12, dtype=np.float64).reshape(2, 1, 6) + 1
    y = pl.rotate_half(x, [0, 3], 4, 100.0, None)
    assert np.allclose(y[0], x[0]) and np.allclose(y[1, 0, 4:], x[1, 0, 4:])
    a = 3 * 0.1                                  # second pair: values 1 and 3 of the head
    assert np.allclose(y[1, 0, [1, 3]], [8 * math.cos(a) - 10 * math.sin(a), 10 * math.cos(a) + 8 * math.sin(a)])
    assert np.allclose(y[1, 0, [0, 2]], [7 * math.cos(3) - 9 * math.sin(3), 9 * math.cos(3) + 7 * math.sin(3)])


def test_plain_lightning_by_hand_and_carried_state():
    rng = np.random.default_rng(0)
    m = dict(heads=2, dim=3, vdim=2, decay=[0.5, 1.0])
    w = {"q": rng.standard_normal((6, 4)), "k": rng.standard_normal((6, 4)), "v": rng.standard_normal((4, 4)),
         "g": rng.standard_normal((4, 4)), "o": rng.standard_normal((4, 4)), "norm": rng.standard_normal(4)}
    h = rng.standard_normal((5, 4))
    out, S = pl.lightning(h, w, m, 1e-6)
    q, k, v = (pl.silu(h @ w[n].T) for n in "qkv")
    o1 = []
    for hd, d in enumerate(m["decay"]):          # token 1 written out: two terms
        kk, vv, qq = k[:, hd * 3:hd * 3 + 3], v[:, hd * 2:hd * 2 + 2], q[1, hd * 3:hd * 3 + 3]
        o1.append(d * (qq @ kk[0]) * vv[0] + (qq @ kk[1]) * vv[1])
    o1 = np.concatenate(o1)
    want = o1 / math.sqrt((o1 ** 2).mean() + 1e-6) * w["norm"] * pl.sigmoid(h[1] @ w["g"].T)
    assert np.allclose(out[1], want @ w["o"].T)
    a, sa = pl.lightning(h[:2], w, m, 1e-6)
    b, sb = pl.lightning(h[2:], w, m, 1e-6, sa)
    assert np.allclose(np.concatenate([a, b]), out) and np.allclose(sb, S)


def test_plain_attention_window_cap_temperature_and_blend_by_hand():
    rng = np.random.default_rng(1)
    m = dict(heads=2, kv_heads=1, dim=4, vdim=3, scale=0.7, softcap=1.5, conv=None, mask=dict(size=3), rot=None, v_mix=True)
    w = {"q": rng.standard_normal((8, 5)), "k": rng.standard_normal((4, 5)), "v": rng.standard_normal((3, 5)),
         "o": rng.standard_normal((5, 6)), "temp": np.array([1.3, 0.6]), "vmix": np.array(0.25)}
    h = rng.standard_normal((6, 5))
    first = rng.standard_normal((6, 1, 3))
    out, own = pl.windowed_attention(h, w, m, first)
    assert np.allclose(own[:, 0], h @ w["v"].T)
    t = 5
    v = 0.75 * (h @ w["v"].T) + 0.25 * first[:, 0]
    heads = []
    for hd in range(2):
        q = h[t] @ w["q"][hd * 4:(hd + 1) * 4].T
        s = np.array([1.5 * math.tanh((q @ (h[j] @ w["k"].T)) * 0.7 * w["temp"][hd] / 1.5) for j in (3, 4, 5)])   # 2 is out
        p = np.exp(s - s.max())
        heads.append((p / p.sum()) @ v[3:6])
    assert np.allclose(out[t], np.concatenate(heads) @ w["o"].T)


def test_plain_depth_average_by_hand(tmp_path):
    """The stream after a layer is the weighted sum of the embedding output and every layer's result; a
    layer's result is its input plus both branches."""
    folder = write_lagedra(str(tmp_path / "m"), LG_A, seed=4)
    plain = pl.PlainLagedra.from_folder(folder)
    toks = [5, 9, 200]
    streams = []
    plain.forward(toks, streams)
    w = plain.w
    x0 = w["embed"][toks] + w["pos"][:3]
    a = pl.scalar_rms_norm(x0, float(w["l0.norm1"]), 1e-5)
    b = pl.scalar_rms_norm(x0, float(w["l0.norm2"]), 1e-5)
    y, own = pl.windowed_attention(a, plain.sub("l0.mix."), LG_A["layers"][0]["mixer"])
    x1 = x0 + y + pl.dense_ffn(b, w["l0.mlp.up"], w["l0.mlp.down"])
    assert np.allclose(streams[0], w["l0.dwa"][0] * x0 + w["l0.dwa"][1] * x1)
    s1 = streams[0]
    x2 = s1 + pl.lightning(pl.scalar_rms_norm(s1, float(w["l1.norm1"]), 1e-5), plain.sub("l1.mix."), LG_A["layers"][1]["mixer"], 1e-5)[0]
    assert np.allclose(streams[1], w["l1.dwa"][0] * x0 + w["l1.dwa"][1] * x1 + w["l1.dwa"][2] * x2)


# ------------------------------------------------------------------ the engine through the stand-ins
def _rel(rows, ref):
    worst = 0.0
    for (rid, p), got in rows.items():
        want = ref[rid][p]
        worst = max(worst, float(np.abs(got - want).max() / max(1e-9, want.std())))
    return worst


@pytest.mark.parametrize("name", list(LG))
def test_engine_on_stand_ins_agrees_with_plain(tmp_path, monkeypatch, name):
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, load_model
    folder = write_lagedra(str(tmp_path / name), LG[name], seed=5)
    plain = pl.PlainLagedra.from_folder(folder)
    reqs = requests_for(LG[name]["vocab"], (1, 7, 70, 33, 150), seed=2)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 12)
    ids = list(reqs)
    for what, steps in (("whole", whole_steps(reqs)), ("one by one", tail_steps(reqs, tail=9)),
                        ("batches", batch_steps(reqs, [ids[:3], ids[3:]])),
                        ("portions", chunk_steps(reqs, [ids[:2], ids[2:]], sizes=(2, 50, 64, 1, 17)))):
        assert _rel(run_steps(eng, steps), ref) < 1e-4, what
    assert not eng.cache.live_slots()


def test_engine_on_stand_ins_random_configuration(tmp_path, monkeypatch):
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, load_model
    raw = random_config(np.random.default_rng(11))
    folder = write_lagedra(str(tmp_path / "r"), raw, seed=6)
    plain = pl.PlainLagedra.from_folder(folder)
    reqs = requests_for(raw["vocab"], (3, 40, 90), seed=4)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 8)
    assert _rel(run_steps(eng, chunk_steps(reqs, [list(reqs)], sizes=(2, 31, 1))), ref) < 1e-4


def test_greedy_generation_on_stand_ins(tmp_path, monkeypatch):
    """`generate` with its scheduler, slots and decode sessions, tokens against the plain model."""
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, generate, load_model
    from minfer_amd.sampling import SamplingParams
    folder = write_lagedra(str(tmp_path / "gen"), LG_C, seed=8)
    plain = pl.PlainLagedra.from_folder(folder)
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 6, max_seqs=2)
    prompts = [[5, 9, 20, 7], [11], [25, 3, 3, 3, 8, 1, 44]]
    res = generate(eng, prompts, SamplingParams(temp=0.0, repeat_penalty=1.0), max_new=5, stop_tokens=[])
    for p, toks in zip(prompts, res.tokens):
        seq = list(p)
        for t in toks:
            assert t == pl.greedy(plain.forward(seq)[-1])
            seq.append(t)
    assert not eng.cache.live_slots()


def test_a_file_may_hold_what_a_layer_has_no_use_for(tmp_path, monkeypatch):
    """The norm before a feed-forward that is not there, the blend of a layer that does not blend."""
    plain_ops.install(monkeypatch)
    from minfer_amd import load_model
    from minfer_amd.weights.safetensors_io import open_model_files, write_safetensors
    folder = write_lagedra(str(tmp_path / "m"), LG_B, seed=3)
    files = open_model_files(folder)
    have = {n: f.tensor(n).clone() for n, f in files.items()}
    have["l2.norm2"] = torch.ones((), dtype=torch.bfloat16)
    have["l1.mix.vmix"] = torch.ones((), dtype=torch.bfloat16)
    del files
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), [(n, tuple(t.shape), t.dtype) for n, t in have.items()],
                      lambda n: have[n])
    with pytest.warns(UserWarning, match="not used"):
        load_model(folder, dtype="float32", device="cpu")


def test_a_cache_entry_with_pages_and_state():
    from minfer_amd.cache.paged import Cache, CacheError, KVRequest, StateRequest
    cache = Cache({0: (KVRequest(2, 8, 5, v_head_dim=3), StateRequest((2, 4))), 1: StateRequest((3,)), 2: None},
                  max_tokens=128, max_seqs=2, dtype=torch.float32, device="cpu")
    k, v, group = cache.kv(0)
    assert tuple(k.shape[1:]) == (2, 64, 8) and tuple(v.shape[1:]) == (2, 64, 3)
    assert tuple(cache.state(0).shape) == (2, 2, 4) and tuple(cache.state(1).shape) == (2, 3)
    s = cache.alloc_slot()
    cache.state(0)[s] = 1.0
    cache.free_slot(s)
    assert cache.alloc_slot() == s and float(cache.state(0)[s].abs().sum()) == 0.0
    with pytest.raises(CacheError):
        Cache({0: (KVRequest(1, 8), KVRequest(1, 8))}, 64, 1, torch.float32, "cpu")
