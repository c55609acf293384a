"""Tabezen on the GPU: each new kernel alone against the plain functions, the engine against the
plain implementation under every way of cutting requests into steps, keys far back and at page
edges that decide the result, long decoding through the captured step, and the programs."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_ops
import plain_tabezen as pt
from replays import batch_steps, chunk_steps, requests_for, run_steps, tail_steps, whole_steps
from tabezen_tiny import TZ, TZ_A, TZ_B, random_config, write_tabezen
from tiny import random_tokens

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# bfloat16 logits against the 64-bit plain implementation, as fractions of the logits' standard
# deviation: this design norms every branch's result, so a layer's roundings are not damped by a
# large residual; measured 1 to 2 % rms at three to five layers
BF16_RMS, BF16_MAX, F32_ABS = 0.04, 0.2, 2e-4
# where the queries are scaled up so that single keys decide the softmax (which is what makes a
# wrong key show), the roundings of the scores are scaled up with them: measured up to 6 % rms at
# single positions; a wrong or missing key there moves a row by its whole size.  The 32-bit run of
# the same case is the sharp instrument.
SHARP = 3.0


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def compare(rows, ref, dtype, what, loosen=1.0, f32_abs=F32_ABS):
    assert rows, "nothing was produced"
    for (rid, p), got in sorted(rows.items()):
        want = ref[rid][p]
        assert np.isfinite(got).all(), f"{what}: non-finite logits at request {rid} position {p}"
        diff = got.astype(np.float64) - want
        if dtype == "float32":
            assert np.abs(diff).max() <= f32_abs * max(1.0, want.std()), \
                f"{what} [float32]: request {rid} position {p} of {len(ref[rid])}: {np.abs(diff).max():.3e}"
        else:
            rms, std = float(np.sqrt(np.mean(diff * diff))), float(want.std())
            assert rms <= loosen * BF16_RMS * std and np.abs(diff).max() <= loosen * BF16_MAX * std, \
                f"{what} [bfloat16]: request {rid} position {p} of {len(ref[rid])}: rms {rms / std:.3f}, max {np.abs(diff).max() / std:.3f}"


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("d, groups", [(96, 3), (200, 1), (1028, 4), (64, 64), (512, 4), (2048, 2), (4096, 1), (256, 256),
                                       (8192, 8)])
def test_group_rmsnorm_kernel(d, groups):
    from minfer_amd.kernels import ops
    x, w = rnd(7, d, seed=1, scale=3.0), rnd(d, seed=2) + 1
    for dtype in (torch.float32, torch.bfloat16):
        want, got = torch.empty(7, d, dtype=dtype), torch.empty(7, d, dtype=dtype, device=DEV)
        plain_ops.group_rmsnorm(x, w, 1e-5, groups, want)
        ops.group_rmsnorm(x.to(DEV), w.to(DEV), 1e-5, groups, got)
        assert (got.cpu().float() - want.float()).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)
    idx = torch.tensor([5, 0, 5], dtype=torch.int32)
    want, got = torch.empty(3, d), torch.empty(3, d, device=DEV)
    plain_ops.group_rmsnorm(x, w, 1e-5, groups, want, idx)
    ops.group_rmsnorm(x.to(DEV), w.to(DEV), 1e-5, groups, got, idx.to(DEV))
    assert (got.cpu() - want).abs().max() < 1e-5
    # added into a stream, with the rounded copy; and in place
    h = rnd(7, d, seed=3)
    want_h, hd = h.clone(), h.to(DEV).clone()
    cast = torch.empty(7, d, dtype=torch.bfloat16, device=DEV)
    plain_ops.group_rmsnorm(x, w, 1e-5, groups, want_h, add=True)
    ops.group_rmsnorm(x.to(DEV), w.to(DEV), 1e-5, groups, hd, add=True, cast_out=cast)
    assert (hd.cpu() - want_h).abs().max() < 1e-5 and torch.equal(cast.cpu(), hd.cpu().to(torch.bfloat16))
    xd = x.to(DEV).clone()
    ops.group_rmsnorm(xd, w.to(DEV), 1e-5, groups, xd)
    want = torch.empty(7, d)
    plain_ops.group_rmsnorm(x, w, 1e-5, groups, want)
    assert (xd.cpu() - want).abs().max() < 1e-5


def test_xielu_kernel():
    from minfer_amd.kernels import ops
    x = torch.cat([rnd(3, 333, seed=4, scale=3.0), torch.tensor([[0.0, -1e-8, 1e-8, -30.0, 30.0] + [0.0] * 328])])
    for dtype in (torch.float32, torch.bfloat16):
        want, got = torch.empty(4, 333, dtype=dtype), torch.empty(4, 333, dtype=dtype, device=DEV)
        plain_ops.xielu(x, want, 0.8, 1.3)
        ops.xielu(x.to(DEV), got, 0.8, 1.3)
        err = ((got.cpu().float() - want.float()).abs() / (1 + want.float().abs())).max()
        assert err < (1e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("m, n, k", [(1, 112, 96), (8, 8192, 2048), (40, 200, 128), (300, 384, 256), (2048, 1000, 136)])
def test_product_with_xielu_epilogue(m, n, k):
    """Every size class of the bfloat16 product (few rows, split K, tiles) with the activation folded in."""
    from minfer_amd.kernels import ops
    x, w = rnd(m, k, seed=1).to(torch.bfloat16), rnd(n, k, seed=2, scale=k ** -0.5).to(torch.bfloat16)
    bias = torch.cat([rnd(n, seed=3, scale=0.5), torch.tensor([0.8, 1.3])])
    want, got = torch.empty(m, n, dtype=torch.bfloat16), torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    plain_ops.linear(x, w, bias, want, xielu=True)
    ops.linear(x.to(DEV), w.to(DEV), bias.to(DEV), got, xielu=True)
    err = ((got.cpu().float() - want.float()).abs() / (1 + want.float().abs())).max()
    assert err < 1e-2


def test_pair_rotation_tables_and_kernel():
    from minfer_amd.kernels import ops
    from minfer_amd.parts.rotary import blended_frequencies
    sc = dict(factor=4.0, original=64, fast=8.0, slow=2.0)
    f, mag = blended_frequencies(12, 500.0, sc)
    f_plain, mag_plain = pt.yarn_frequencies(12, 500.0, sc)
    assert np.allclose(f, f_plain, rtol=1e-14) and mag == mag_plain
    cs, sn = ops.rope_table_freqs(3000, f, mag, DEV)
    pos = np.arange(3000)[:, None] * np.asarray(f)[None, :]
    assert np.abs(cs.cpu().numpy() - np.cos(pos) * mag).max() < 1e-6
    assert np.abs(sn.cpu().numpy() - np.sin(pos) * mag).max() < 1e-6
    x = rnd(5, 4 * 16, seed=5)
    positions = torch.tensor([0, 1, 70, 2999, 64], dtype=torch.int32)
    got = x.to(DEV).clone()
    ops.rope_pairs_inplace(got, cs, sn, positions.to(DEV), 3, 4, 16)
    want = x.double().view(5, 4, 16).numpy().copy()
    want[:, :3] = pt.rotate_interleaved(want[:, :3], positions.numpy(), 12, 500.0, sc)
    assert np.abs(got.cpu().numpy().reshape(5, 4, 16) - want).max() < 1e-5


@pytest.mark.parametrize("w, lens", [(80, (1, 5, 200, 64, 129)), (300, (700,)), (257, (3, 128, 65))])
def test_mingru_scan_kernels(w, lens):
    """Both forms of the scan against the plain walk, over ragged sequences, twice in a row with
    the state carried and the slots in another order than the sequences."""
    from minfer_amd.kernels import ops
    slots = torch.tensor([4, 0, 2, 5, 1][:len(lens)], dtype=torch.int32)
    state_ref = rnd(6, w, seed=6)
    state_a, state_b = state_ref.to(DEV).clone(), state_ref.to(DEV).clone()
    for rnd_no in range(2):
        n = sum(lens)
        zug = rnd(n, 3 * w, seed=7 + rnd_no, scale=2.0)
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
        want = torch.empty(n, w)
        plain_ops.mingru_scan(zug, cu, slots, state_ref, want)
        a, b = torch.empty(n, w, device=DEV), torch.empty(n, w, device=DEV)
        ops.mingru_scan(zug.to(DEV), cu.to(DEV), slots.to(DEV), state_a, a)
        ops.mingru_scan(zug.to(DEV), cu.to(DEV), slots.to(DEV), state_b, b, ops.scan_chunks(list(lens)).to(DEV))
        for got, st in ((a, state_a), (b, state_b)):
            assert (got.cpu() - want).abs().max() < 2e-5
            assert (st.cpu() - state_ref).abs().max() < 2e-5
    assert torch.equal(state_a[3], state_ref[3].to(DEV)) or len(lens) > 3      # a slot no sequence uses is untouched


def test_headwise_linear_kernel():
    from minfer_amd.kernels import ops
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        x = rnd(11, 3, 50, seed=8).to(dtype)
        wt = rnd(3, 37, 290, seed=9, scale=0.2).to(dtype)
        gate = torch.rand(11, 3, generator=torch.Generator().manual_seed(1))
        want = torch.zeros(11, 3, 300, dtype=dtype)
        plain_ops.headwise_linear(x, 37, wt, want, 290, gate)
        got = torch.zeros(11, 3, 300, dtype=dtype, device=DEV)
        ops.headwise_linear(x.to(DEV), 37, wt.to(DEV), got, 290, gate.to(DEV))
        assert (got.cpu().float() - want.float()).abs().max() < tol
        assert got[:, :, 290:].abs().max() == 0


@pytest.mark.parametrize("n_tok, heads, n_in, n_out, stride", [(11, 3, 40, 290, 48), (1, 16, 128, 512, 128),
                                                              (100, 5, 72, 8, 72), (8, 2, 264, 40, 264),
                                                              (300, 3, 128, 500, 136), (1000, 2, 512, 120, 512),
                                                              (257, 4, 40, 90, 48)])
def test_headwise_linear_matrix_core_kernel(n_tok, heads, n_in, n_out, stride):
    from minfer_amd.kernels import ops
    x = rnd(n_tok, heads, stride, seed=8).to(torch.bfloat16)
    wo = rnd(heads, n_out, n_in, seed=9, scale=0.2).to(torch.bfloat16)
    gate = torch.rand(n_tok, heads, generator=torch.Generator().manual_seed(1))
    for g in (None, gate):
        want = torch.zeros(n_tok, heads, n_out + 4, dtype=torch.bfloat16)
        plain_ops.headwise_linear_mfma(x, n_in, wo, want, n_out, g)
        got = torch.zeros(n_tok, heads, n_out + 4, dtype=torch.bfloat16, device=DEV)
        ops.headwise_linear_mfma(x.to(DEV), n_in, wo.to(DEV), got, n_out, None if g is None else g.to(DEV))
        assert ((got.cpu().float() - want.float()).abs() / (1 + want.float().abs())).max() < 1e-2
        assert got[:, :, n_out:].abs().max() == 0


def _latent_case(dtype, heads, rank, rot, lens, seed, needle=None):
    """Cached rows for sequences of `lens` tokens in shuffled pages of a NaN-poisoned pool, queries
    for the last few positions of each.  `needle` = (sequence, position): that row is made to
    decide the softmax of the sequence's queries."""
    dk = rank + rot
    n_pages = sum((n + 63) // 64 for n in lens) + 3
    cache = torch.full((n_pages, 1, 64, dk), float("nan"), dtype=dtype)
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    cols = max((n + 63) // 64 for n in lens)
    table = torch.full((len(lens), cols), -1, dtype=torch.int32)
    flat = cache.view(n_pages, 64, dk)
    for b, n in enumerate(lens):
        rows = rnd(n, dk, seed=seed + b)
        if needle and needle[0] == b:
            rows[needle[1]] *= 6.0
        for p in range((n + 63) // 64):
            table[b, p] = order.pop()
            m = min(64, n - p * 64)
            flat[table[b, p], :m] = rows[p * 64:p * 64 + m].to(dtype)
    seq, pos = [], []
    for b, n in enumerate(lens):
        for p in sorted({0, n // 2, max(0, n - 2), n - 1} | ({63, 64, 65} & set(range(n)))):
            seq.append(b)
            pos.append(p)
    q = rnd(len(seq), heads, dk, seed=seed + 50, scale=0.5)
    if needle:
        b, p = needle
        for i, s in enumerate(seq):
            if s == b:
                q[i] = flat[table[b, p // 64], p % 64].float()[None, :] * 0.5 + 0.05 * q[i]
    return cache, table, torch.tensor(seq, dtype=torch.int32), torch.tensor(pos, dtype=torch.int32), q.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, rank, rot, window", [(3, 40, 8, 0), (5, 72, 16, 0), (2, 264, 4, 0), (1, 24, 16, 70)])
def test_latent_attention_kernel_far_keys_and_page_edges(dtype, heads, rank, rot, window):
    from minfer_amd.kernels import ops
    lens = (1, 64, 65, 700, 130)
    for needle in (None, (3, 5), (3, 63), (3, 64), (4, 128)):
        if window and needle:
            continue
        cache, table, seq, pos, q = _latent_case(dtype, heads, rank, rot, lens, seed=11, needle=needle)
        want = torch.empty(len(seq), heads, rank, dtype=dtype)
        plain_ops.latent_attn(q, cache, table, pos, seq, want, rank, 0.35, window, max(lens))
        got = torch.empty(len(seq), heads, rank, dtype=dtype, device=DEV)
        ops.latent_attn(q.to(DEV), cache.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), got, rank, 0.35, window,
                        max(lens))
        assert torch.isfinite(got).all()
        err = (got.cpu().float() - want.float()).abs().max()
        assert err < (2e-5 if dtype == torch.float32 else 4e-2), f"needle {needle}: {err}"
        if needle:      # the needle's row is what comes out for the queries behind it
            b, p = needle
            row = cache.view(-1, 64, rank + rot)[table[b, p // 64], p % 64, :rank].float()
            for i in range(len(seq)):
                if seq[i] == b and pos[i] >= p:
                    assert (got[i].cpu().float() - row[None, :]).abs().max() < 0.15 * row.abs().max()


def _step_context(lens, new, table):
    """The ragged layout of a step in which sequence b (of lens[b] tokens) brings its last new[b]."""
    from minfer_amd.engine.batch import StepContext
    start = [n - k for n, k in zip(lens, new)]
    seq = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(new)).int()
    pos = torch.cat([torch.arange(s, s + k) for s, k in zip(start, new)]).int()
    cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32)
    return StepContext(cache=None, n_tokens=sum(new), n_seqs=len(lens), token_ids=torch.zeros(sum(new), dtype=torch.int32, device=DEV),
                       positions=pos.to(DEV), seq_of_tok=seq.to(DEV), cu_seqlens=cu.to(DEV),
                       start_pos=torch.tensor(start, dtype=torch.int32, device=DEV),
                       slot_ids=torch.arange(len(lens), dtype=torch.int32, device=DEV), logit_rows=None,
                       page_tables={0: table.to(DEV)}, max_len=max(lens), max_new=max(new),
                       all_decode=all(k == 1 for k in new), host_new=list(new), host_start=start), seq, pos


@pytest.mark.parametrize("heads, rank, rot, window", [(3, 40, 8, 0), (5, 72, 16, 0), (2, 264, 8, 0), (1, 24, 16, 70),
                                                      (16, 64, 32, 0), (70, 32, 8, 0)])
@pytest.mark.parametrize("new", [(1, 64, 65, 700, 130), (1, 1, 1, 1, 1), (1, 2, 40, 33, 129)])
def test_latent_attention_matrix_core_kernel(heads, rank, rot, window, new):
    """The matrix-core kernel on ragged steps (whole prompts, one token each, portions on top of
    a context) over shuffled pages of a NaN-poisoned pool, with and without a row that decides."""
    from minfer_amd.kernels import ops
    lens = (1, 64, 65, 700, 130)
    assert ops.latent_mfma_takes(torch.bfloat16, rank, rank + rot)
    for needle in (None, (3, 5), (3, 64), (4, 127)):
        if window and needle:
            continue
        cache, table, _, _, _ = _latent_case(torch.bfloat16, heads, rank, rot, lens, seed=13, needle=needle)
        ctx, seq, pos = _step_context(lens, new, table)
        q = rnd(len(seq), heads, rank + rot, seed=60, scale=0.5)
        if needle:
            b, p = needle
            row = cache.view(-1, 64, rank + rot)[table[b, p // 64], p % 64].float()
            for i in range(len(seq)):
                if seq[i] == b:
                    q[i] = row[None, :] * 0.5 + 0.05 * q[i]
        q = q.to(torch.bfloat16)
        want = torch.empty(len(seq), heads, rank, dtype=torch.bfloat16)
        plain_ops.latent_attn(q, cache, table, pos, seq, want, rank, 0.35, window, max(lens))
        got = torch.full((len(seq), heads, rank), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.latent_attn(q.to(DEV), cache.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), got, rank, 0.35, window,
                        max(lens), ctx=ctx)
        assert torch.isfinite(got).all()
        err = (got.cpu().float() - want.float()).abs().max()
        assert err < 4e-2, f"needle {needle}: {err}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_prep_kernel(dtype):
    from minfer_amd.kernels import ops
    from minfer_amd.parts.rotary import blended_frequencies
    H, dn, dr, rank, rd = 3, 10, 8, 20, 6
    f, mag = blended_frequencies(rd, 100.0, None)
    cs, sn = plain_ops.rope_table_freqs(300, f, mag, "cpu")
    lens, start = (5, 70), (60, 0)
    seq = torch.tensor([0] * 5 + [1] * 70, dtype=torch.int32)
    pos = torch.tensor(list(range(60, 65)) + list(range(70)), dtype=torch.int32)
    table = torch.tensor([[2, 0], [3, 1]], dtype=torch.int32)
    ld = H * (dn + dr) + rank + dr + H + 3
    proj = rnd(75, ld, seed=12)
    w = rnd(rank, seed=13) + 1
    outs = []
    for side in ("plain", "gpu"):
        dev = "cpu" if side == "plain" else DEV
        cache = torch.zeros(4, 1, 64, rank + dr, dtype=dtype, device=dev)
        qp = torch.empty(75, H, dn, dtype=dtype, device=dev)
        qa = torch.zeros(75, H, rank + dr, dtype=dtype, device=dev)
        gate = torch.empty(75, H, device=dev)
        fn = plain_ops.latent_prep if side == "plain" else ops.latent_prep
        fn(proj.to(dev), H * (dn + dr), H * (dn + dr) + rank + dr, w.to(dev), 1e-5, cs.to(dev), sn.to(dev), pos.to(dev),
           seq.to(dev), table.to(dev), cache, qp, qa, gate, H, dn, dr, rank, True)
        outs.append([t.cpu().float() for t in (cache, qp, qa, gate)])
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    for a, b in zip(*outs):
        assert (a - b).abs().max() < tol


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("tabezen")
    return {name: write_tabezen(str(tmp / name), raw, seed=i) for i, (name, raw) in enumerate(TZ.items())}


@pytest.fixture(scope="module")
def plains(folders):
    return {name: pt.PlainTabezen.from_folder(f) for name, f in folders.items()}


def engine_for(folder, dtype, max_tokens=64 * 16, **kw):
    from minfer_amd import Engine, load_model
    return Engine(load_model(folder, dtype=dtype, device="cuda:0"), max_tokens=max_tokens, poison_cache=True, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TZ))
def test_replays_agree_with_plain(folders, plains, name, dtype):
    """Whole; the last tokens one by one; unequal batches one after another (slots and pages used
    again); prompts in portions down to two tokens and one, alone and in mixed batches."""
    reqs = requests_for(TZ[name]["vocab"], (1, 7, 64, 150, 65, 33, 300), seed=3)
    ref = {rid: plains[name].forward(toks) for rid, toks in reqs.items()}
    ids = list(reqs)
    eng = engine_for(folders[name], dtype)
    lo = SHARP if name == "B" else 1.0
    compare(run_steps(eng, whole_steps(reqs)), ref, dtype, f"{name} whole", lo)
    compare(run_steps(eng, tail_steps(reqs, tail=40)), ref, dtype, f"{name} last 40 one by one", lo)
    compare(run_steps(eng, batch_steps(reqs, [ids[:4], ids[4:]])), ref, dtype, f"{name} unequal batches", lo)
    compare(run_steps(eng, chunk_steps(reqs, [ids[:3], ids[3:]])), ref, dtype, f"{name} portions in batches", lo)
    compare(run_steps(eng, chunk_steps(reqs, [[r] for r in ids], sizes=(2,))), ref, dtype, f"{name} portions of 2", lo)
    compare(run_steps(eng, chunk_steps(reqs, [[r] for r in ids], sizes=(129, 3, 64))), ref, dtype, f"{name} portions of 129", lo)
    assert not eng.cache.live_slots()


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whatever config.json may say: sizes, orders and options drawn at random, both run types,
    whole, one by one, in batches and in portions."""
    raw = random_config(np.random.default_rng(2000 + seed))
    folder = write_tabezen(str(tmp_path / "m"), raw, seed=seed)
    plain = pt.PlainTabezen.from_folder(folder)
    reqs = requests_for(raw["vocab"], (1, 9, 70, 200, 131), seed=seed)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    ids = list(reqs)
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(folder, dtype)
        what = f"random configuration {seed} ({json.dumps(raw)[:300]})"
        compare(run_steps(eng, whole_steps(reqs)), ref, dtype, what + " whole", SHARP)
        compare(run_steps(eng, tail_steps(reqs, tail=33)), ref, dtype, what + " one by one", SHARP)
        compare(run_steps(eng, batch_steps(reqs, [ids[:3], ids[3:]])), ref, dtype, what + " batches", SHARP)
        compare(run_steps(eng, chunk_steps(reqs, [ids[:2], ids[2:]])), ref, dtype, what + " portions", SHARP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_with_sharp_attention_and_long_decoding(tmp_path, dtype):
    """Queries scaled so that the softmax picks single keys, many of them hundreds of positions
    back: a prompt of 900 tokens whole, then again as 800 + 100 one by one."""
    # in 32-bit the queries are doubled on top of the configuration's own sharp scale (the roundings of
    # the scores grow with them: 1e-3 instead of 2e-4); bfloat16 keeps the configuration's scale
    folder = write_tabezen(str(tmp_path / "sharp"), TZ_B, seed=21, sharpen=2.0 if dtype == "float32" else 1.0)
    plain = pt.PlainTabezen.from_folder(folder)
    reqs = {"long": random_tokens(512, 900, 77)}
    ref = {"long": plain.forward(reqs["long"])}
    eng = engine_for(folder, dtype, max_tokens=64 * 16)
    compare(run_steps(eng, whole_steps(reqs)), ref, dtype, "sharp whole", SHARP, 1e-3)
    compare(run_steps(eng, tail_steps(reqs, tail=100)), ref, dtype, "sharp 800 + 100 one by one", SHARP, 1e-3)


def test_greedy_generation_through_the_entry_point(folders, plains):
    """`LLM.generate`: the scheduler, slots used again (more prompts than slots), the captured decode
    step; 70 new tokens so that every sequence crosses a page edge while decoding."""
    from minfer_amd import LLM
    llm = LLM(folders["A"], dtype="float32", n_ctx=256, n_slots=2)
    prompts = [random_tokens(300, n, 30 + i) for i, n in enumerate((5, 60, 1, 17))]
    res = llm.generate(prompts, max_new=70, temp=0.0, repeat_penalty=1.0, stop_tokens=[])
    eager = llm.generate(prompts, max_new=70, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False)
    assert res.tokens == eager.tokens
    for p, toks in zip(prompts, res.tokens):
        assert len(toks) == 70
        seq = list(p)
        logits = plains["A"].forward(seq + toks)
        for i, t in enumerate(toks):
            row = logits[len(p) + i - 1]
            top = np.sort(row)[-2:]
            assert t == pt.greedy(row) or top[1] - top[0] < 1e-4, f"token {i}"
    bf = LLM(folders["A"], dtype="bfloat16", n_ctx=256, n_slots=4)
    a = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[]).tokens
    b = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False).tokens
    assert a == b


def test_programs(folders, plains, tmp_path):
    """bin/minfer generates greedily from a Tabezen folder; bin/trace_run replays a batch."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "minfer"), folders["C"], "--prompt-tokens", "5,6,7;9",
                        "--greedy", "--repeat-penalty", "1.0", "-n", "4", "--dtype", "float32", "--n-ctx", "64",
                        "--stop-token", "100000"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.strip().splitlines() if l]
    for line, prompt in zip(lines, ([5, 6, 7], [9])):
        seq = list(prompt)
        for t in (int(x) for x in line.split(",")):
            assert t == pt.greedy(plains["C"].forward(seq)[-1])
            seq.append(t)
    reqs = requests_for(97, (3, 70, 20), seed=9)
    ref = {rid: plains["C"].forward(toks) for rid, toks in reqs.items()}
    steps = batch_steps(reqs, [list(reqs)])
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["C"], "--dtype",
                          "float32", "--out", out, "--max-tokens", "93"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                         text=True, bufsize=1)
    rows, pos = {}, {}
    try:
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            assert p.stdout.readline().strip() == f"done {st['step']}"
            arr = np.fromfile(os.path.join(out, f"{st['step']}.f32"), dtype="<f4").reshape(-1, 97)
            i = 0
            for e in st["entries"]:
                for w in e["want"]:
                    rows[(e["id"], pos.get(e["id"], 0) + w)] = arr[i]
                    i += 1
                pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()
    compare(rows, ref, "float32", "trace_run")
