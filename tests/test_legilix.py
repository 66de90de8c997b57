"""Legilix (pre-norm layer-list model with grouped RMS norms: windowed
softmax attention with q/k norm, half rotary and pre-softmax score mixing, or
with a logarithmic distance bias and an output gate; GELU MLP or sigmoid-routed
experts with scaled input) against the plain oracle in legilix_oracle.py.

Every test builds its own small configuration and random weights. The
``dev`` fixture runs each case on the CPU path and, marked ``gpu``, on the
HIP kernels (fp32 and bf16 models).
"""

import json
import math
import os
import subprocess
import sys

import pytest
import torch

import legilix_oracle as O
from distrl_llm_amd.config import EngineConfig, SamplingParams
from distrl_llm_amd.engine.hybrid_engine import HybridEngine
from distrl_llm_amd.models.hybrid import (HybridLM, legilix_config_from_spec,
                                          legilix_spec_from_config,
                                          rotary_frequencies,
                                          save_legilix_checkpoint)
from distrl_llm_amd.ops import seqmix as SM

CASES = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
         pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
         pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.fixture(params=CASES)
def dev(request):
    return request.param


def tol(dtype):
    # bf16 is a coarse check of a deep, narrow model (its rounding noise on
    # the logits is a few percent); the same kernels are held to 2e-4 in fp32
    # and the bf16-only tiled kernel has tests of its own
    return 2e-4 if dtype == torch.float32 else 0.12


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    return float(d.pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-9))


def mixed_cfg():
    """Both mixers twice with sizes unequal wherever the design allows: 1, 2
    and 3 query heads per kv head, rotated part below and equal to the head
    size, with and without frequency rescaling, windows with and without
    kept tokens and no window at all, dense and expert feed-forwards (top 1,
    2 and all) and a layer without one."""
    return O.make_cfg([
        O.rotary_layer(heads=4, kv_heads=2, dim=8, vdim=6, window=7, keep=2, rot_dims=4,
                       mlp=(5, 2, 10)),
        O.distance_layer(heads=6, kv_heads=2, dim=4, vdim=10, window=5, mlp=12),
        O.rotary_layer(heads=3, kv_heads=3, dim=6, vdim=5, window=9, keep=0, rot_dims=6,
                       scaling=None, base=50.0, mlp=None),
        O.distance_layer(heads=2, kv_heads=1, dim=8, vdim=8, window=0, mlp=(3, 3, 8)),
        O.rotary_layer(heads=2, kv_heads=1, dim=12, vdim=4, window=0, keep=0, rot_dims=2,
                       mlp=(4, 1, 6)),
    ], width=24, vocab=37, groups=3)


def build(cfg, dev, seed=0, blocks=64, block_size=4, slots=4, W=None):
    device, dtype = dev
    W = W if W is not None else O.random_weights(cfg, seed)
    model = HybridLM(legilix_spec_from_config(cfg), dtype=dtype, device=device)
    model.load_tensors(W)
    eng = HybridEngine(model, EngineConfig(max_seq_length=4096, kv_block_size=block_size,
                                           num_kv_blocks=blocks, num_state_slots=slots,
                                           max_num_seqs=slots), device=torch.device(device))
    return W, eng


def run_portions(eng, tokens, cuts, capture=None):
    q = eng.open_sequence()
    out, at = [], 0
    for n in cuts:
        out.append(eng.step([(q, tokens[at:at + n])], [list(range(n))], capture=capture))
        at += n
    assert at == len(tokens)
    eng.close_sequence(q)
    return torch.cat(out)


def toks(n, vocab, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def ints(v, device):
    return torch.tensor(v, dtype=torch.int32, device=device)


# ------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("groups", [1, 2, 5])
def test_grouped_norm_and_residual(dev, groups):
    device, dtype = dev
    g = torch.Generator().manual_seed(0)
    T, D, eps = 5, 40, 1e-4
    x = torch.randn(T, D, generator=g)
    x[:, :D // groups] *= 20.0                  # one group much larger than the rest
    y = torch.randn(T, D, generator=g).to(dtype).float()
    w = 1.0 + 0.3 * torch.randn(D, generator=g)
    h32, hb = SM.offset_rmsnorm(x.to(device), w.to(device), eps, dtype, 0.0, groups)
    assert rel_err(h32, O.group_norm(x.double(), w.double(), groups, eps)) < 1e-6
    assert hb.dtype == dtype
    for nxt in (w, None):
        xd = x.clone().to(device)
        h = SM.residual_add_norm(xd, y.to(dtype).to(device),
                                 None if nxt is None else nxt.to(device), eps, dtype, 0.0, groups)
        s = x.double() + y.double()
        assert rel_err(xd, s) < 1e-6
        if nxt is None:
            assert h is None
        else:
            assert h.dtype == dtype
            assert rel_err(h.float(), O.group_norm(s, w.double(), groups, eps)) < (
                1e-6 if dtype == torch.float32 else 5e-3)


def test_gelu(dev):
    device, dtype = dev
    z = torch.linspace(-6, 6, 97).view(1, -1).to(dtype)
    got = SM.gelu_tanh(z.to(device))
    assert got.dtype == dtype
    assert rel_err(got.float(), O.gelu_tanh(z.double())) < (1e-6 if dtype == torch.float32 else 5e-3)


def test_rotary_table():
    for dims, base, sc in ((4, 100.0, (4.0, 16, 2.0, 0.5)), (6, 50.0, None),
                           (10, 3000.0, (16.0, 64, 8.0, 1.0)), (2, 10.0, (2.0, 8, 1.0, 1.0))):
        rot = {"dims": dims, "base": base}
        if sc:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), sc))
        f, mag = rotary_frequencies(dims, base, sc)
        fo, mo = O.rotary_table(rot)
        assert f == pytest.approx(fo, rel=1e-12) and mag == pytest.approx(mo, rel=1e-12)


@pytest.mark.parametrize("H,G,dk,dv,rot_dims,norm,mix", [
    (4, 2, 8, 6, 4, True, True), (3, 3, 6, 5, 6, True, False), (6, 2, 10, 3, 0, False, False),
    (2, 1, 12, 4, 2, False, True), (5, 1, 72, 8, 70, True, True)])
def test_qk_prepare(dev, H, G, dk, dv, rot_dims, norm, mix):
    """Norm, rotation of part of each head, fold of the mixing matrix and
    page write, from strided projection rows with columns to spare."""
    device, dtype = dev
    g = torch.Generator().manual_seed(2)
    T, eps, extra = 7, 1e-3, 5
    need = (H + G) * dk + G * dv
    wide = torch.randn(T, need + extra, generator=g).to(dtype)
    qw = 1.0 + 0.3 * torch.randn(dk, generator=g)
    kw = 1.0 + 0.3 * torch.randn(dk, generator=g)
    M = torch.eye(H) + 0.4 * torch.randn(H, H, generator=g)
    rot = {"dims": rot_dims, "base": 77.0,
           "scaling": dict(factor=3.0, original=12, fast=2.0, slow=0.5)}
    pos = [11, 0, 3, 200, 4, 5, 1]
    slot = [9, 2, 0, 5, 11, 3, 7]
    freqs, mag = None, 1.0
    if rot_dims:
        f, mag = rotary_frequencies(rot_dims, 77.0, (3.0, 12.0, 2.0, 0.5))
        freqs = torch.tensor(f, dtype=torch.float64).float().to(device)
    cache = torch.zeros(12, G * (dk + dv), dtype=dtype, device=device)
    got = SM.qk_prepare_kv_write(
        wide.to(device)[:, :need + 2], H, G, dk, dv, qw.to(device) if norm else None,
        kw.to(device) if norm else None, eps, ints(pos, device), freqs, mag,
        M.to(device) if mix else None, ints(slot, device), cache)
    x = wide.double()
    q, k = x[:, :H * dk].view(T, H, dk), x[:, H * dk:(H + G) * dk].view(T, G, dk)
    if norm:
        q, k = O.head_norm(q, qw.double(), eps), O.head_norm(k, kw.double(), eps)
    q = torch.stack([O.rotate_halves(q[t], pos[t], rot) for t in range(T)])
    k = torch.stack([O.rotate_halves(k[t], pos[t], rot) for t in range(T)])
    bound = 1e-5 if dtype == torch.float32 else 6e-3
    rows = cache[torch.tensor(slot).to(device)].float().cpu()
    assert rel_err(rows[:, :G * dk], k.reshape(T, -1)) < bound
    assert torch.equal(rows[:, G * dk:], wide[:, (H + G) * dk:need].float())
    if mix:
        rep = H // G
        want = torch.zeros(T, H, G, dk, dtype=torch.float64)
        for h in range(H):
            for a in range(H):
                want[:, h, a // rep] += M[h, a].double() * q[:, a]
        assert tuple(got.shape) == (T, H, G * dk)
        assert rel_err(got.float(), want.reshape(T, H, G * dk)) < bound
    else:
        assert tuple(got.shape) == (T, H, dk)
        assert rel_err(got.float(), q) < bound


def _attention_case(device, dtype, H, G, dk, dv, bs, lengths, news, seed=0, kd=None):
    """A paged cache filled with random keys and values for rows of the given
    lengths, whose last ``news`` tokens are the step's queries."""
    g = torch.Generator().manual_seed(seed)
    W = G * (dk + dv)
    nblk = sum((n + bs - 1) // bs for n in lengths)
    perm = torch.randperm(nblk, generator=g).tolist()
    cache = torch.zeros((nblk + 1) * bs, W, dtype=dtype, device=device)
    tables, kv, qs, pos, seq, cu = [], [], [], [], [], [0]
    for b, (n, m) in enumerate(zip(lengths, news)):
        nb = (n + bs - 1) // bs
        tables.append([perm.pop() for _ in range(nb)])
        rows = torch.randn(n, W, generator=g).to(dtype)
        kv.append(rows.float())
        idx = torch.tensor([tables[-1][j // bs] * bs + j % bs for j in range(n)])
        cache[idx.to(device)] = rows.to(device)
        qs.append(torch.randn(m, H, kd or dk, generator=g).to(dtype))
        pos += list(range(n - m, n))
        seq += [b] * m
        cu.append(cu[-1] + m)
    width = max(len(t) for t in tables)
    tables = [t + [0] * (width - len(t)) for t in tables]
    return cache, tables, kv, torch.cat(qs), pos, seq, cu


def _softmax_direct(q, kv, pos, seq, H, G, dk, dv, whole, scale, window, keep, r1, r2, gate):
    out = torch.zeros(q.shape[0], H, dv, dtype=torch.float64)
    for t in range(q.shape[0]):
        rows, p = kv[seq[t]].double(), pos[t]
        js = O.visible(p, {"size": window, "keep_first": keep})
        for a in range(H):
            gi = a // (H // G)
            keys = rows[js, :G * dk] if whole else rows[js, gi * dk:(gi + 1) * dk]
            s = (keys @ q[t, a].double()) * scale
            if r1 is not None:
                d = torch.tensor([float(p - j) for j in js], dtype=torch.float64)
                s = s - r1[a] * torch.log(1.0 + r2[a] * d)
            o = torch.softmax(s, -1) @ rows[js, G * dk + gi * dv:G * dk + (gi + 1) * dv]
            out[t, a] = o if gate is None else o / (1.0 + math.exp(-float(gate[t, a])))
    return out.reshape(q.shape[0], H * dv)


def _run_attention(device, dtype, H, G, dk, dv, whole, window, keep, dist, gated, bs, lengths,
                   news, seed=0):
    kd = G * dk if whole else dk
    cache, tables, kv, q, pos, seq, cu = _attention_case(device, dtype, H, G, dk, dv, bs,
                                                         lengths, news, seed, kd)
    g = torch.Generator().manual_seed(seed + 100)
    r1 = (0.5 + torch.rand(H, generator=g)) if dist else None
    r2 = (0.2 + torch.rand(H, generator=g)) if dist else None
    # the gate is a column slice of a wider matrix, as in the model
    gwide = torch.randn(q.shape[0], H + 3, generator=g).to(dtype) if gated else None
    tiles, mt = SM.query_tiles(news, SM.WIDE_QUERY_TILE)
    got = SM.window_attention(
        q.to(device), cache, H, G, dk, dv, whole, ints(tables, device), bs, ints(cu, device),
        ints(seq, device), ints(pos, device), 0.31, window, keep,
        None if r1 is None else r1.to(device), None if r2 is None else r2.to(device),
        None if gwide is None else gwide.to(device)[:, 2:2 + H], dtype,
        tiles=ints(tiles, device), max_tile=mt)
    want = _softmax_direct(q.float(), kv, pos, seq, H, G, dk, dv, whole, 0.31, window, keep,
                           r1, r2, None if gwide is None else gwide[:, 2:2 + H].float())
    return got, want


@pytest.mark.parametrize("H,G,dk,dv,whole,window,keep,dist,gated", [
    (4, 2, 6, 5, True, 5, 2, False, False), (3, 3, 8, 7, True, 7, 0, False, False),
    (6, 2, 4, 10, False, 5, 0, True, True), (2, 1, 8, 8, False, 0, 0, True, True),
    (6, 2, 16, 24, True, 9, 12, False, True), (5, 5, 7, 3, False, 4, 1, True, False)])
def test_window_attention_op(dev, H, G, dk, dv, whole, window, keep, dist, gated):
    """Prompt portions and single tokens in one step against a direct
    softmax: own or whole key rows, with and without distance bias and gate,
    a kept range longer than the window, pages in random order."""
    device, dtype = dev
    got, want = _run_attention(device, dtype, H, G, dk, dv, whole, window, keep, dist, gated,
                               4, [23, 9, 14, 1], [11, 1, 14, 1])
    assert rel_err(got.float(), want) < (1e-5 if dtype == torch.float32 else 6e-3)


def test_window_attention_edges(dev):
    """One key made to stand out (a score far above the rest, a value of its
    own): it must take the whole softmax just inside the window, among the
    kept first tokens and at page borders, and must not count just outside
    either, from a prompt portion and from a single decoded token."""
    device, dtype = dev
    H, G, dk, dv, bs, window, keep = 2, 1, 8, 8, 4, 12, 3
    n = 40
    mark = torch.arange(1, dv + 1).float()
    for m in (1, 9):                                   # decoded token / portion
        p = n - 1                                      # the last query's position
        for j_star, seen in ((p - window + 1, True), (p - window, False), (keep - 1, True),
                             (keep, False), (0, True), (p, True), (p - 4, True), (p - 3, True)):
            g = torch.Generator().manual_seed(3)
            kvr = 0.05 * torch.randn(n, dk + dv, generator=g)
            kvr[j_star, :dk] = 4.0
            kvr[j_star, dk:] = mark
            kvr = kvr.to(dtype)
            q = torch.full((m, H, dk), 4.0).to(dtype)  # q.k* * scale = 64 above the rest
            nb = (n + bs - 1) // bs
            table = list(range(nb - 1, -1, -1))
            cache = torch.zeros((nb + 1) * bs, dk + dv, dtype=dtype, device=device)
            idx = torch.tensor([table[j // bs] * bs + j % bs for j in range(n)])
            cache[idx.to(device)] = kvr.to(device)
            pos = list(range(n - m, n))
            tiles, mt = SM.query_tiles([m], SM.WIDE_QUERY_TILE)
            got = SM.window_attention(
                q.to(device), cache, H, G, dk, dv, False, ints([table], device), bs,
                ints([0, m], device), ints([0] * m, device), ints(pos, device), 0.5, window,
                keep, None, None, None, dtype, tiles=ints(tiles, device), max_tile=mt)
            last = got[-1].float().cpu().view(H, dv)
            if seen:
                assert rel_err(last[0], mark.double()) < 2e-2, (m, j_star)
            else:
                assert float(last.abs().max()) < 0.2, (m, j_star)


def test_far_key_among_hundreds(dev):
    """Without a window a key 600 tokens back, across many pages, must still
    be found by a decoded token and by the last token of a portion."""
    device, dtype = dev
    H, G, dk, dv, bs, n = 4, 2, 8, 8, 16, 640
    for m in (1, 70):
        g = torch.Generator().manual_seed(5)
        kvr = 0.05 * torch.randn(n, G * (dk + dv), generator=g)
        j_star = 37
        kvr[j_star, :G * dk] = 4.0
        kvr[j_star, G * dk:] = torch.arange(1, G * dv + 1).float()
        kvr = kvr.to(dtype)
        q = torch.full((m, H, dk), 4.0).to(dtype)
        nb = (n + bs - 1) // bs
        table = torch.randperm(nb, generator=g).tolist()
        cache = torch.zeros((nb + 1) * bs, G * (dk + dv), dtype=dtype, device=device)
        idx = torch.tensor([table[j // bs] * bs + j % bs for j in range(n)])
        cache[idx.to(device)] = kvr.to(device)
        tiles, mt = SM.query_tiles([m], SM.WIDE_QUERY_TILE)
        got = SM.window_attention(
            q.to(device), cache, H, G, dk, dv, False, ints([table], device), bs,
            ints([0, m], device), ints([0] * m, device), ints(list(range(n - m, n)), device),
            0.5, 0, 0, None, None, None, dtype, tiles=ints(tiles, device), max_tile=mt)
        last = got[-1].float().cpu().view(H, dv)
        for a in range(H):
            want = torch.arange(1, dv + 1).double() + (a // 2) * dv
            assert rel_err(last[a], want) < 2e-2, (m, a)


@pytest.mark.parametrize("E,top,ff", [(5, 2, 10), (3, 3, 8), (4, 1, 6), (1, 1, 4)])
def test_router_and_scaled_experts(dev, E, top, ff):
    """Sigmoid scores, no renormalisation, the weight on the expert's input."""
    device, dtype = dev
    g = torch.Generator().manual_seed(4)
    T, D = 9, 24
    fc = {"router": {"experts": E, "top": top}}
    w = {"router": torch.randn(E, D, generator=g)}
    for e in range(E):
        for nm, shape in (("gate", (ff, D)), ("up", (ff, D)), ("down", (D, ff))):
            w[f"e{e}.{nm}"] = (torch.randn(*shape, generator=g) / math.sqrt(shape[1])
                               ).to(torch.bfloat16).float()
    h = torch.randn(T, D, generator=g).to(dtype)
    gu = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)])
    down = torch.stack([w[f"e{e}.down"] for e in range(E)])
    idx, wts = SM.moe_route_sigmoid(h.to(device), w["router"].to(device), top)
    for t in range(T):
        oi, ow = O.route(w, "", h[t].double(), top)
        assert idx[t].tolist() == oi
        assert torch.allclose(wts[t].double().cpu(), torch.stack(ow), atol=1e-6)
    got = SM.moe_experts_scaled_input(h.to(device), idx, wts, gu.to(dtype).to(device),
                                      down.to(dtype).to(device))
    want = O.moe_ff(fc, w, "", h.double())
    assert rel_err(got, want) < (1e-5 if dtype == torch.float32 else 1.5e-2)


# ------------------------------------------------------------ whole models

@pytest.mark.parametrize("which", ["rotary", "distance"])
def test_single_layer_models(dev, which):
    layer = (O.rotary_layer(mlp=None) if which == "rotary" else O.distance_layer(mlp=None))
    cfg = O.make_cfg([layer], width=24, vocab=31, groups=2)
    W, eng = build(cfg, dev)
    t = toks(25, 31, seed=3)
    assert rel_err(run_portions(eng, t, [25]), O.forward(cfg, W, t)) < tol(dev[1])
    assert rel_err(run_portions(eng, t, [9] + [1] * 16), O.forward(cfg, W, t)) < tol(dev[1])


def test_whole_prompt_and_layers(dev):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    t = toks(45, 37, seed=4)
    lay, cap = [], []
    want = O.forward(cfg, W, t, lay)
    got = run_portions(eng, t, [45], capture=cap)
    assert len(cap) == len(lay) == 5
    for i, (a, b) in enumerate(zip(cap, lay)):
        assert rel_err(a, b) < tol(dev[1]), i
    assert rel_err(got, want) < tol(dev[1])


def test_first_tokens(dev):
    """Sequences of one, two and three tokens, alone and token by token."""
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    for n in (1, 2, 3):
        t = toks(n, 37, seed=5 + n)
        want = O.forward(cfg, W, t)
        assert rel_err(run_portions(eng, t, [n]), want) < tol(dev[1])
        assert rel_err(run_portions(eng, t, [1] * n), want) < tol(dev[1])


@pytest.mark.parametrize("cuts", [[1] * 30, [2] * 15, [7, 2, 2, 1, 11, 3, 4], [16, 14], [29, 1],
                                  [3, 27]])
def test_portions(dev, cuts):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    t = toks(30, 37, seed=6)
    assert rel_err(run_portions(eng, t, cuts), O.forward(cfg, W, t)) < tol(dev[1])


def test_portions_do_not_change_fp32_results(dev):
    if dev[1] != torch.float32:
        pytest.skip("fp32 statement")
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    t = toks(40, 37, seed=7)
    whole = run_portions(eng, t, [40])
    for cuts in ([1] * 40, [2] * 20, [13, 5, 2, 20], [39, 1]):
        assert rel_err(run_portions(eng, t, cuts), whole) < 2e-5


def test_mixed_batches_and_reuse(dev):
    """Unequal requests in one step (portions beside single tokens, requests
    sitting steps out), pages and slots given back and taken again; every
    position against the oracle and against the request run alone."""
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=40, slots=3)
    V = 37
    reqs = {k: toks(n, V, seed=10 + i) for i, (k, n) in
            enumerate((("a", 26), ("b", 9), ("c", 17), ("d", 22), ("e", 5)))}
    plan = [[("a", 7), ("b", 2)], [("a", 1), ("b", 3), ("c", 9)], [("a", 1), ("c", 2)],
            [("a", 6), ("b", 4), ("c", 1)], [("c", 5), ("a", 1)], [("a", 10), ("d", 3)],
            [("d", 1), ("e", 2)], [("d", 12), ("e", 1)], [("d", 6), ("e", 2)]]
    live, at, got = {}, {k: 0 for k in reqs}, {k: [] for k in reqs}
    for stepn in plan:
        work, want = [], []
        for k, n in stepn:
            if k not in live:
                live[k] = eng.open_sequence()
            work.append((live[k], reqs[k][at[k]:at[k] + n]))
            want.append(list(range(n)))
        out = eng.step(work, want)
        o = 0
        for k, n in stepn:
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
            if at[k] == len(reqs[k]):
                eng.close_sequence(live.pop(k))
    assert not live
    _, solo = build(cfg, dev, W=W)
    for k, t in reqs.items():
        g = torch.cat(got[k])
        assert rel_err(g, O.forward(cfg, W, t)) < tol(dev[1]), k
        alone = run_portions(solo, t, [len(t)])
        assert rel_err(g, alone) < (1e-5 if dev[1] == torch.float32 else 0.06), k


def test_dirty_pages_and_slots(dev):
    """Freed pages hold another request's leftovers."""
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=12, slots=1)
    a, b = toks(40, 37, seed=20), toks(35, 37, seed=21)
    run_portions(eng, a, [40])
    for r in eng.pool.rows.values():
        r.add_(5.0)
    assert rel_err(run_portions(eng, b, [20, 15]), O.forward(cfg, W, b)) < tol(dev[1])
    assert eng.pool.allocator.num_free == 12 and eng.slots.num_free == 1


def test_long_decode_past_windows(dev):
    """120 single-token steps: every window passes over decoded tokens, the
    kept first tokens stay."""
    cfg = O.make_cfg([O.rotary_layer(window=9, keep=3, mlp=8),
                      O.distance_layer(window=11, mlp=(4, 2, 6)),
                      O.rotary_layer(heads=2, kv_heads=2, window=16, keep=5, mlp=None)],
                     width=16, vocab=31, groups=2)
    W, eng = build(cfg, dev, blocks=48)
    t = toks(132, 31, seed=30)
    got = run_portions(eng, t, [12] + [1] * 120)
    want = O.forward(cfg, W, t)
    assert rel_err(got, want) < tol(dev[1])
    assert rel_err(got[-20:], want[-20:]) < tol(dev[1])


@pytest.mark.parametrize("which", ["rotary", "distance"])
def test_window_edges_in_model(dev, which):
    """Moving the token just inside a window, or the last kept one, changes a
    later position's logits; the token just outside both does not."""
    device, dtype = dev
    if which == "rotary":
        layer, probes = O.rotary_layer(window=6, keep=2, mlp=None), (
            (19 - 5, True), (19 - 6, False), (1, True), (2, False))
    else:
        layer, probes = O.distance_layer(window=6, mlp=None), (
            (19 - 5, True), (19 - 6, False), (0, False))
    cfg = O.make_cfg([layer], width=16, vocab=31, groups=1)
    W, eng = build(cfg, dev)
    base = toks(20, 31, seed=40)
    ref = run_portions(eng, base, [10] + [1] * 10)[-1]
    for j, seen in probes:
        alt = list(base)
        alt[j] = (alt[j] + 7) % 31
        for cuts in ([20], [10] + [1] * 10, [13, 2, 5]):
            out = run_portions(eng, alt, cuts)[-1]
            moved = rel_err(out, ref)
            assert (moved > 1e-3) == seen, (j, cuts, moved)
            assert rel_err(out, O.forward(cfg, W, alt)[-1]) < tol(dtype)


def test_other_sizes(dev):
    """Values a model may happen to make equal or 1: one head, one kv head,
    one norm group, one expert, window 1, rotation over the whole head, unit
    scales, every size equal."""
    cfg = O.make_cfg([
        O.rotary_layer(heads=1, kv_heads=1, dim=8, vdim=8, window=1, keep=1, rot_dims=8,
                       scaling=None, scale=1.0, mlp=8),
        O.distance_layer(heads=1, kv_heads=1, dim=8, vdim=8, window=1, scale=1.0, mlp=(1, 1, 8)),
        O.rotary_layer(heads=8, kv_heads=8, dim=8, vdim=8, window=8, keep=8, rot_dims=8,
                       mlp=(8, 8, 8)),
        O.distance_layer(heads=8, kv_heads=1, dim=8, vdim=8, window=8, mlp=8),
    ], width=8, vocab=11, groups=1, embed_scale=1.0, logit_scale=1.0)
    W, eng = build(cfg, dev)
    t = toks(21, 11, seed=50)
    want = O.forward(cfg, W, t)
    assert rel_err(run_portions(eng, t, [21]), want) < tol(dev[1])
    assert rel_err(run_portions(eng, t, [5, 2, 1, 13]), want) < tol(dev[1])
    cfg = O.make_cfg([O.rotary_layer(heads=6, kv_heads=3, dim=10, vdim=14, window=3, keep=5,
                                     rot_dims=10, mlp=(7, 3, 5))],
                     width=30, vocab=19, groups=30)          # every entry its own group
    W, eng = build(cfg, dev)
    t = toks(19, 19, seed=51)
    assert rel_err(run_portions(eng, t, [6, 13]), O.forward(cfg, W, t)) < tol(dev[1])


def test_greedy_generate(dev):
    """Greedy decoding through generate() and its scheduler (small step
    budget, two prompts): every generated token is the oracle's argmax for
    its prefix wherever the oracle's margin is not a rounding matter."""
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=64, slots=4)
    eng.cfg.step_token_budget = 8
    prompts = [toks(13, 37, seed=60), toks(6, 37, seed=61)]
    sp = SamplingParams(max_tokens=10, temperature=0.0, n=1)
    outs = eng.generate(prompts, sp)
    margin = 1e-3 if dev[1] == torch.float32 else 0.3
    for p, o in zip(prompts, outs):
        gen = o[0]
        assert len(gen) == 10
        logits = O.forward(cfg, W, p + gen)
        for i, tok in enumerate(gen):
            row = logits[len(p) - 1 + i]
            top2 = torch.topk(row, 2).values
            if float(top2[0] - top2[1]) > margin:
                assert int(row.argmax()) == tok, (i, tok)
    assert eng.slots.num_free == 4 and eng.pool.allocator.num_free == 64


def test_fork_shares_pages(dev):
    """n-candidate fan-out: the fork shares the prompt's full pages and gets
    a copy of the partial page of every attention layer."""
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=20, block_size=4)
    t = toks(18, 37, seed=33)
    q = eng.open_sequence()
    eng.step([(q, t[:10])], [[]])
    c = eng.fork_sequence(q)
    tail2 = [(x + 3) % 37 for x in t[10:]]
    out = eng.step([(q, t[10:]), (c, tail2)], [list(range(8)), list(range(8))])
    assert rel_err(out[:8], O.forward(cfg, W, t)[10:]) < tol(dev[1])
    assert rel_err(out[8:], O.forward(cfg, W, t[:10] + tail2)[10:]) < tol(dev[1])
    eng.close_sequence(q)
    eng.close_sequence(c)
    assert eng.pool.allocator.num_free == 20


def test_served_through_the_batcher():
    """The server's app, batcher and sampler drive the design's engine like
    any other: greedy completions repeat, sampled ones fan out."""
    from fastapi.testclient import TestClient

    from distrl_llm_amd.serve import create_app
    from distrl_llm_amd.utils.tokenizer import ByteTokenizer
    cfg = O.make_cfg([O.rotary_layer(mlp=8), O.distance_layer(mlp=(4, 2, 6))],
                     width=16, vocab=600, groups=4)
    _, eng = build(cfg, ("cpu", torch.float32), blocks=128, block_size=8, slots=8)
    client = TestClient(create_app(eng, ByteTokenizer(vocab_size=600), "tiny-legilix"))
    body = {"prompt": "2+2=", "max_tokens": 5, "temperature": 0.0}
    a = client.post("/v1/completions", json=body).json()
    b = client.post("/v1/completions", json=body).json()
    assert a["choices"][0]["text"] == b["choices"][0]["text"]
    assert a["usage"]["completion_tokens"] <= 5
    r = client.post("/v1/completions", json={"prompt": ["abcd", "wxyz"], "max_tokens": 3,
                                             "temperature": 1.0, "top_p": 0.9, "n": 2}).json()
    assert len(r["choices"]) == 4
    assert eng.pool.allocator.num_free == 128 and eng.slots.num_free == 8


@pytest.mark.gpu
def test_captured_decode_matches_eager():
    cfg = mixed_cfg()
    dev = ("cuda", torch.bfloat16)
    W, eng = build(cfg, dev)
    _, eager = build(cfg, dev, W=W)
    eager.cfg.enforce_eager = True
    t = toks(30, 37, seed=70)
    a = run_portions(eng, t, [10] + [1] * 20)
    b = run_portions(eager, t, [10] + [1] * 20)
    assert rel_err(a, b) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv,whole,window,keep,dist,gated,lengths,news", [
    (4, 2, 64, 64, True, 100, 9, False, False, [300, 70, 129], [200, 70, 65]),
    (8, 2, 32, 48, False, 50, 0, True, True, [333, 64], [333, 5]),
    (4, 4, 128, 128, False, 0, 0, True, False, [257], [257]),
    (8, 2, 80, 40, True, 150, 12, False, True, [500, 21], [260, 21]),
    (16, 4, 128, 128, True, 200, 4, False, False, [450], [300]),
    (2, 1, 8, 8, True, 30, 40, True, True, [150, 90], [100, 90]),
])
def test_tiled_window_attention_kernel(H, G, dk, dv, whole, window, keep, dist, gated, lengths,
                                       news):
    """The bf16 MFMA kernel against a direct softmax in float64: several key
    widths (up to 512 folded columns), value widths, windows whose edges fall
    inside tiles and blocks, kept ranges longer than the window."""
    got, want = _run_attention("cuda", torch.bfloat16, H, G, dk, dv, whole, window, keep, dist,
                               gated, 16, lengths, news, seed=7)
    assert rel_err(got.float(), want) < 6e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dk,dv,whole,window,keep,dist,lengths", [
    (8, 2, 64, 64, True, 300, 16, False, [700, 40, 1, 333]),
    (4, 4, 32, 16, False, 0, 0, True, [1500, 9]),
    (6, 1, 16, 24, False, 64, 0, True, [64, 65, 63, 200]),
    (8, 1, 8, 8, True, 70, 100, False, [400, 90]),
    (3, 1, 40, 8, False, 128, 8, False, [129, 135, 140]),
])
def test_grouped_window_attention_kernel(dtype, H, G, dk, dv, whole, window, keep, dist, lengths):
    """Decode steps (one token per row) through the grouped kernel and its
    merge of key shares: head ratios 1-8, shares with and without blocks."""
    got, want = _run_attention("cuda", dtype, H, G, dk, dv, whole, window, keep, dist, True, 16,
                               lengths, [1] * len(lengths), seed=9)
    assert rel_err(got.float(), want) < (1e-5 if dtype == torch.float32 else 6e-3)


# --------------------------------------------------- files, registry, tools

def test_checkpoint_registry_and_replay(tmp_path):
    """Save a checkpoint, load it through the registry, replay a step trace
    with the command-line tool and compare with the oracle."""
    from distrl_llm_amd.models.registry import hybrid_design_of, load_model_and_engine
    cfg = mixed_cfg()
    W = O.random_weights(cfg, 3)
    model = HybridLM(legilix_spec_from_config(cfg), dtype=torch.float32, device="cpu")
    model.load_tensors(W)
    assert legilix_spec_from_config(legilix_config_from_spec(model.spec)) == model.spec
    path = str(tmp_path / "tiny")
    save_legilix_checkpoint(model, path)
    assert hybrid_design_of(path) == "legilix"
    m2, eng = load_model_and_engine(path, EngineConfig(max_seq_length=256, kv_block_size=4,
                                                       num_kv_blocks=32, num_state_slots=2,
                                                       max_num_seqs=2),
                                    dtype=torch.float32, device=torch.device("cpu"))
    for k, v in model.export_tensors().items():
        assert torch.equal(v, m2.export_tensors()[k]), k
    a, b = toks(21, 37, seed=80), toks(11, 37, seed=81)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [8]},
                                     {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [0, 8]},
                                     {"id": "a", "tokens": a[9:10], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[10:], "want": [10]}], "end": ["a"]}]
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path,
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == [
        "done 0", "done 1", "done 2"]
    import numpy as np
    la, lb = O.forward(cfg, W, a), O.forward(cfg, W, b)
    want = {0: la[8:9], 1: torch.stack([lb[2], lb[10], la[9]]), 2: la[20:21]}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, 37))
        assert rel_err(got, w) < 2e-4, n


def test_config_errors():
    good = mixed_cfg()
    legilix_spec_from_config(good)

    def broken(change):
        cfg = json.loads(json.dumps(good))
        change(cfg)
        with pytest.raises((ValueError, KeyError)):
            legilix_spec_from_config(cfg)

    broken(lambda c: c["layers"][0].update(type="attention_3"))
    broken(lambda c: c["layers"][0]["mixer"].update(kv_heads=3))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=5))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10))
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=9))
    broken(lambda c: c["layers"][1]["mlp"].update(kind="glu"))
    broken(lambda c: c["norm"].update(groups=5))
    broken(lambda c: c["layers"][1]["mixer"].pop("scale"))
