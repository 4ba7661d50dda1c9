"""Gibavik through the engine, and its kernels alone, against the plain restatement in oracle/gibavik_oracle.py.

Every test makes its own small configuration and weights.  The engine is built on a directory that holds config.json (and,
where the weights are made by the test, model.safetensors), as a user's would be; steps are given with Engine.run_given (the
replay entry point) or chosen by the scheduler (Engine.step / LLM.generate).  Comparisons are in float32 unless a test says
otherwise: there a structural fault (a key too many, a window one token off, a lost state) stands far above rounding.
"""
import asyncio
import json
import os

import numpy as np
import pytest
import torch

from oracle import gibavik_oracle as go
from seq_drivers import F32_TOL, close, cuts_of, greedy, make_engine, model_dir, replay, step_layout, tokens

pytestmark = pytest.mark.gpu

LEFT = {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 20, "mask": {"size": 9}, "rot": {"dims": 8, "base": 500.0}, "scale": 0.3, "softcap": 7.0}
RIGHT = {"heads": 3, "dim": 10, "vdim": 12, "decay": [0.5, 0.9, 0.995]}
MOE2 = {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 2}}
MOE1 = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 3, "top": 1}}
DENSE = {"kind": "dense", "ff": 50, "limit": 1.5}
PAR = {"type": "parallel", "mixer": {"left": LEFT, "right": RIGHT, "left_scale": 0.7, "right_scale": 1.3}, "mlp": MOE2}
ATT = {"type": "attention", "mixer": {"heads": 6, "kv_heads": 2, "dim": 12, "vdim": 28, "scale": 0.2}, "mlp": DENSE}


def borrowing(layer, src, mlp=MOE1):
    m = dict(layer["mixer"], kv_from=src)
    return {"type": "attention", "mixer": m, "mlp": mlp}


def make_cfg(layers, width=40, vocab=61, eps=1e-5, emb=3.0, cap=9.0):
    return {"architecture": "Gibavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": emb}, "logit_softcap": cap,
            "layers": json.loads(json.dumps(layers))}


def weights_of(cfg, seed=0):
    """The weights an engine built on a directory without a checkpoint draws for `seed`."""
    from nano_vllm_x_amd.gibavik import GibavikConfig, random_checkpoint
    return dict(random_checkpoint(GibavikConfig.from_dict(cfg), seed))


def forward(cfg, w, toks):
    return go.forward(cfg, w, toks)


# ---- kernels alone -------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [70, 1, 300])
def test_normed_results_are_added_to_the_stream(fmt, width):
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(width)
    t = 5
    x = torch.randn(t, width, generator=g)
    y, y2 = (torch.randn(t, width, generator=g).to(fmt) for _ in range(2))
    one, per, nxt = torch.tensor([1.7]), torch.randn(width, generator=g), torch.tensor([0.6])
    tol = 1e-5 if fmt == torch.float32 else 2e-2
    # one result, one number as the weight; the next sublayer reads the stream itself
    xd = x.cuda()
    h = ops.postnorm_residual(xd, y=y.cuda(), w_post=one.cuda(), eps=1e-3)
    want = x + go.scalar_norm(y.float(), one, 1e-3)
    assert torch.allclose(xd.cpu(), want, atol=1e-5) and h.dtype == fmt and torch.allclose(h.float().cpu(), want, atol=tol)
    # two results weighted and summed before the norm, a weight per channel, and the closing norm on the new stream
    xd = x.cuda()
    h = ops.postnorm_residual(xd, y=y.cuda(), y2=y2.cuda(), a=0.7, b=1.3, w_post=per.cuda(), eps=1e-3, w_next=nxt.cuda())
    want = x + go.unit_rms(0.7 * y.float() + 1.3 * y2.float(), 1e-3) * per
    assert torch.allclose(xd.cpu(), want, atol=1e-5) and torch.allclose(h.float().cpu(), go.scalar_norm(want, nxt, 1e-3), atol=tol)
    # the closing norm alone leaves the stream as it is
    xd = x.cuda()
    h = ops.postnorm_residual(xd, w_next=per.cuda(), eps=1e-3, out_dtype=fmt)
    assert torch.equal(xd.cpu(), x) and torch.allclose(h.float().cpu(), go.unit_rms(x, 1e-3) * per, atol=tol)


def test_scaled_embedding_and_capped_logits():
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(0)
    table = torch.randn(31, 70, generator=g)
    ids = torch.tensor([3, 30, 0, 3], dtype=torch.int64)
    for fmt in (torch.float32, torch.bfloat16):
        x, h = ops.embed_scale(ids.cuda(), table.to(fmt).cuda(), 12.5)
        assert x.dtype == torch.float32 and h.dtype == fmt
        assert torch.equal(x.cpu(), table.to(fmt).float()[ids] * 12.5) and torch.equal(h.cpu(), (table.to(fmt).float()[ids] * 12.5).to(fmt))
    z = torch.randn(4, 70, generator=g) * 30
    assert torch.allclose(ops.tanh_cap(z.cuda(), 11.0).cpu(), 11.0 * torch.tanh(z / 11.0), atol=1e-5)
    assert torch.equal(ops.tanh_cap(z.to(torch.bfloat16).cuda(), 0.0).cpu(), z.to(torch.bfloat16).float())


@pytest.mark.parametrize("mode", ["head", "row", "none"])
@pytest.mark.parametrize("interleaved", [False, True])
def test_query_key_norms_rotation_and_rotated_values(mode, interleaved):
    """Positions up to several thousand; the rotated part is a leading part of a head (or all of it); the values are turned over
    their whole size; rows are a slice of a wider projection; a negative slot stores nothing; a layer without keys of its own."""
    from nano_vllm_x_amd import ops
    from nano_vllm_x_amd.layers.rotary_embedding import rotary_frequencies
    g = torch.Generator().manual_seed(5)
    t, heads, kvh, dim, vdim, rot, base = 6, 3, 1, 22, 10, 6, 3000.0
    nq, nk, nv = heads * dim, kvh * dim, kvh * vdim
    x = torch.randn(t, 5 + nq + nk + nv + 7, generator=g)
    pos = torch.tensor([0, 1, 17, 4095, 5000, 2], dtype=torch.int64)
    slots = torch.tensor([4, 0, -1, 7, 2, 5], dtype=torch.int64)
    qw, kw = (torch.randn(dim if mode == "head" else n, generator=g) for n in (nq, nk))
    freq, vfreq = rotary_frequencies(rot, base)[0], rotary_frequencies(vdim, base)[0]
    kc, vc = torch.full((8, nk), 9.0).cuda(), torch.full((8, nv), 9.0).cuda()
    q, turn = ops.attn_prep_store(x.cuda(), (5, 5 + nq, 5 + nq + nk), pos.cuda(), qw.cuda(), kw.cuda(), mode, 1e-4, freq.cuda(), rot, interleaved,
                                  vfreq.cuda(), slots.cuda(), kc, vc, heads, kvh, dim, vdim)
    ang = pos.double()[:, None] * vfreq[None, :]
    assert torch.allclose(turn.cpu().double(), torch.cat([torch.cos(ang), torch.sin(ang)], dim=1), atol=1e-6)
    xq, xk, xv = x[:, 5:5 + nq].double(), x[:, 5 + nq:5 + nq + nk].double(), x[:, 5 + nq + nk:5 + nq + nk + nv].double()
    if mode == "head":
        xq, xk = go.unit_rms(xq.view(t, heads, dim), 1e-4) * qw, go.unit_rms(xk.view(t, kvh, dim), 1e-4) * kw
    elif mode == "row":
        xq, xk = (go.unit_rms(xq, 1e-4) * qw).view(t, heads, dim), (go.unit_rms(xk, 1e-4) * kw).view(t, kvh, dim)
    else:
        xq, xk = xq.view(t, heads, dim), xk.view(t, kvh, dim)
    wq = go.turn(xq, pos, base, rot, interleaved).reshape(t, nq)
    wk = go.turn(xk, pos, base, rot, interleaved).reshape(t, nk)
    wv = go.turn(xv.view(t, kvh, vdim), pos, base, vdim, interleaved).reshape(t, nv)
    assert torch.allclose(q.cpu().double(), wq, atol=2e-5)
    keep = slots >= 0
    assert torch.allclose(kc.cpu().double()[slots[keep]], wk[keep], atol=2e-5) and torch.allclose(vc.cpu().double()[slots[keep]], wv[keep], atol=2e-5)
    untouched = [s for s in range(8) if s not in slots.tolist()]
    assert (kc.cpu()[untouched] == 9.0).all() and (vc.cpu()[untouched] == 9.0).all()
    # queries only: nothing is read or written for keys and values
    q2, none = ops.attn_prep_store(x.cuda(), (5, 0, 0), pos.cuda(), qw.cuda(), None, mode, 1e-4, freq.cuda(), rot, interleaved, None, None, None, None,
                                   heads, 0, dim, vdim)
    assert torch.equal(q2, q) and none is None


def _cached(keys, values, n_slots, seed):
    """Per-sequence keys (T, G, D) and values (T, G, E) put at scattered slots of caches; returns caches and each sequence's slots."""
    perm = torch.randperm(n_slots, generator=torch.Generator().manual_seed(seed)).tolist()
    g, d, e = keys[0].shape[1], keys[0].shape[2], values[0].shape[2]
    kc, vc = torch.zeros(n_slots, g * d), torch.zeros(n_slots, g * e)
    lists = []
    for k, v in zip(keys, values):
        s = [perm.pop() for _ in range(k.shape[0])]
        kc[s], vc[s] = k.reshape(len(s), -1), v.reshape(len(s), -1)
        lists.append(s)
    return kc, vc, lists


def _turn_table(totals, lens, freq):
    """cos | sin of position * freq for every token of a step, as attn_prep_store hands them to the attention."""
    pos = torch.cat([torch.arange(n - l, n) for n, l in zip(totals, lens)]).double()
    ang = pos[:, None] * freq.double().cpu()[None, :]
    return torch.cat([torch.cos(ang), torch.sin(ang)], dim=1).float().cuda()


def _attend(ops, q_rows, lens, totals, lists, kc, vc, fmt, decode, vfreq=None, **kw):
    """ops.softcap_attn for a step that brings the last lens[b] tokens of the first totals[b] of sequence b."""
    if vfreq is not None:
        kw["v_turn"] = _turn_table(totals, lens, vfreq)
    flat = torch.tensor([s for b, l in enumerate(lists) for s in l[:totals[b]]], dtype=torch.int32).cuda()
    start = torch.tensor(np.concatenate([[0], np.cumsum(totals)[:-1]]), dtype=torch.int64).cuda()
    kv_len = torch.tensor(totals, dtype=torch.int32).cuda()
    lay = step_layout(ops, lens, [n - l for n, l in zip(totals, lens)], list(range(len(lens))), decode)
    return ops.softcap_attn(q_rows.to(fmt).cuda(), kc.to(fmt).cuda(), vc.to(fmt).cuda(), flat, start, kv_len, lay, **kw).float().cpu()


@pytest.mark.parametrize("window", [0, 1, 5, 64, 70])
@pytest.mark.parametrize("penalty", [False, True])
def test_attention_window_and_distance_penalty(window, penalty):
    """Two sequences of unequal length at scattered slots, portions and single tokens, with and without the key split.  One key per
    query stands out (scaled query and key): the one just OUTSIDE the window, which must not be seen, or the very first one
    (far away) where there is no window."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(window + 7)
    heads, kvh, dim, vdim, scale, cap = 4, 2, 16, 24, 0.3, 11.0
    n = [200, 77]
    q = [torch.randn(t, heads, dim, generator=g) for t in n]
    k = [torch.randn(t, kvh, dim, generator=g) for t in n]
    v = [torch.randn(t, kvh, vdim, generator=g) for t in n]
    for b in range(2):                                   # query i asks loudly for key i - window (or key 0)
        for i in range(n[b]):
            j = i - window if window and i >= window else 0
            for h in range(heads):
                kj = k[b][j, h // (heads // kvh)]
                q[b][i, h] = 5.0 * kj / kj.norm()
    r1 = torch.tensor([0.9, 0.0, 0.3, 2.0]) if penalty else None
    r2 = torch.tensor([0.5, 3.0, 0.01, 1.0]) if penalty else None
    want = [go.attend(q[b].double(), k[b].double(), v[b].double(), scale, cap=cap, window=window or None, r1=r1, r2=r2) for b in range(2)]
    kc, vc, lists = _cached(k, v, 300, 3)
    kw = dict(scale=scale, cap=cap, heads=heads, kv_heads=kvh, dim=dim, vdim=vdim, window=window, r1=r1.cuda() if penalty else None,
              r2=r2.cuda() if penalty else None)
    for lens, totals, decode in (([200, 77], [200, 77], False), ([3, 70], [131, 77], False), ([1, 1], [66, 65], True), ([1, 1], [200, 2], True),
                                 ([2, 1], [2, 1], False)):
        rows = torch.cat([q[b][totals[b] - lens[b]:totals[b]].reshape(lens[b], -1) for b in range(2)])
        ref = torch.cat([want[b][totals[b] - lens[b]:totals[b]].reshape(lens[b], -1) for b in range(2)])
        for split in (1, 4):
            got = _attend(ops, rows, lens, totals, lists, kc, vc, torch.float32, decode, n_split=split, **kw)
            close(got, ref, 1e-4, f"lens {lens} of {totals}, split {split}")
    got = _attend(ops, torch.cat([x.reshape(x.shape[0], -1) for x in q]), n, n, lists, kc, vc, torch.bfloat16, False, **kw)
    close(got, torch.cat([x.reshape(x.shape[0], -1) for x in want]), 6e-2, "bfloat16")
    # the restatement itself depends on the edge: a window one key wider sees the loud key
    if window:
        wider = go.attend(q[0].double(), k[0].double(), v[0].double(), scale, cap=cap, window=window + 1, r1=r1, r2=r2)
        assert (wider[window:] - want[0][window:]).abs().max() > 0.1


@pytest.mark.parametrize("dim,vdim", [(64, 96), (96, 64), (128, 128)])
@pytest.mark.parametrize("window", [0, 5, 70])
@pytest.mark.parametrize("interleaved", [False, True])
def test_attention_on_the_matrix_cores(dim, vdim, window, interleaved):
    """Steps of many tokens in bfloat16 take the tile kernel (64 queries of a sequence per workgroup, keys in tiles of 32): ragged
    prompts that end in the middle of a tile, portions that start in the middle of one, a loud key just outside every window, the
    distance penalty, the read-out turned back and gated; against the restatement on the same bfloat16 values, and against the
    vector kernel."""
    from nano_vllm_x_amd import ops
    from nano_vllm_x_amd.layers.rotary_embedding import rotary_frequencies
    g = torch.Generator().manual_seed(dim + window)
    heads, kvh, scale, cap, base = 4, 2, 0.2, 9.0, 300.0
    n = [200, 77, 300, 1]
    bf = lambda x: x.to(torch.bfloat16).float()
    q = [bf(torch.randn(t, heads, dim, generator=g)) for t in n]
    k = [bf(torch.randn(t, kvh, dim, generator=g)) for t in n]
    v = [bf(torch.randn(t, kvh, vdim, generator=g)) for t in n]
    for b in range(len(n)):
        for i in range(n[b]):
            j = i - window if window and i >= window else 0
            for h in range(heads):
                kj = k[b][j, h // (heads // kvh)]
                q[b][i, h] = bf(4.0 * kj / kj.norm())
    gate = [bf(torch.randn(t, heads * vdim, generator=g)) for t in n]
    r1, r2 = torch.tensor([0.9, 0.0, 0.3, 2.0]), torch.tensor([0.5, 3.0, 0.01, 1.0])
    want = []
    for b in range(len(n)):
        pos = torch.arange(n[b])
        turned = bf(go.turn(v[b].double(), pos, base, vdim, interleaved).float())            # values are cached turned, in bfloat16
        v[b] = turned
        o = go.attend(q[b].double(), k[b].double(), turned.double(), scale, cap=cap, window=window or None, r1=r1, r2=r2)
        want.append(go.turn(o, pos, base, vdim, interleaved, sign=-1.0).reshape(n[b], -1) * torch.sigmoid(gate[b].double()))
    kc, vc, lists = _cached(k, v, 700, 5)
    vfreq = rotary_frequencies(vdim, base)[0].cuda()
    kw = dict(scale=scale, cap=cap, heads=heads, kv_heads=kvh, dim=dim, vdim=vdim, window=window, r1=r1.cuda(), r2=r2.cuda(), vfreq=vfreq,
              v_interleaved=interleaved, n_split=1)
    assert ops._lib.load().nvx_softcap_attn_tile_fits(0, dim, vdim, int(not interleaved)) == 1
    for lens, totals in ((n, n), ([70, 3, 130, 1], [200, 77, 300, 1]), ([129, 77, 1, 1], [130, 77, 65, 1])):
        rows = torch.cat([q[b][totals[b] - lens[b]:totals[b]].reshape(lens[b], -1) for b in range(len(n))])
        gates = torch.cat([gate[b][totals[b] - lens[b]:totals[b]] for b in range(len(n))]).to(torch.bfloat16).cuda()
        ref = torch.cat([want[b][totals[b] - lens[b]:totals[b]] for b in range(len(n))])
        tile = _attend(ops, rows, lens, totals, lists, kc, vc, torch.bfloat16, False, gate=gates, matrix_cores=True, **kw)
        vec = _attend(ops, rows, lens, totals, lists, kc, vc, torch.bfloat16, False, gate=gates, matrix_cores=False, **kw)
        for got, what in ((tile, "matrix cores"), (vec, "vector units")):
            # results are bfloat16: half a unit in the last place is 2^-9 of the value; a wrong key would move them by tenths
            err = ((got.double() - ref).abs() / (ref.abs() + 0.05 * ref.std())).max().item()
            assert err < 8e-3, f"{what}, lens {lens} of {totals}: {err:.2e}"


@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("vdim", [20, 64, 130])
def test_read_out_is_turned_back_and_gated(interleaved, vdim):
    from nano_vllm_x_amd import ops
    from nano_vllm_x_amd.layers.rotary_embedding import rotary_frequencies
    g = torch.Generator().manual_seed(vdim)
    heads, kvh, dim, base = 2, 1, 8, 200.0
    n = 40
    q, k, v = torch.randn(n, heads, dim, generator=g), torch.randn(n, kvh, dim, generator=g), torch.randn(n, kvh, vdim, generator=g)
    gate = torch.randn(n, heads * vdim + 3, generator=g)
    pos = torch.arange(n)
    turned = go.turn(v.double(), pos, base, vdim, interleaved)
    o = go.attend(q.double(), k.double(), turned, 0.4)
    want = go.turn(o, pos, base, vdim, interleaved, sign=-1.0).reshape(n, -1) * torch.sigmoid(gate[:, 3:].double())
    kc, vc, lists = _cached([k], [turned.float()], 50, 1)
    vfreq = rotary_frequencies(vdim, base)[0].cuda()
    kw = dict(scale=0.4, cap=0.0, heads=heads, kv_heads=kvh, dim=dim, vdim=vdim, vfreq=vfreq, v_interleaved=interleaved, gate=gate.cuda()[:, 3:])
    for split in (1, 3):
        got = _attend(ops, q.reshape(n, -1), [n], [n], lists, kc, vc, torch.float32, False, n_split=split, **kw)
        close(got, want, 1e-4, f"prompt, split {split}")
    kw["gate"] = gate.cuda()[n - 1:, 3:]
    got = _attend(ops, q[n - 1:].reshape(1, -1), [1], [n], lists, kc, vc, torch.float32, True, **kw)
    close(got, want[n - 1:], 1e-4, "single token")


@pytest.mark.parametrize("dim,vdim", [(10, 12), (70, 5), (32, 64), (1, 1)])
def test_decayed_memory_continues_over_cuts_and_reused_slots(dim, vdim):
    """Two sequences in slots that are not in order, cut into steps of 1, 2 and more tokens; a third sequence later takes over a
    used slot and must start from zero.  A decay close to one keeps the first token for hundreds of steps."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(dim)
    heads = 3
    decay = [0.6, 0.9975, 1.0]
    hd, he = heads * dim, heads * vdim
    full = {0: torch.randn(130, 2 + 2 * hd + he, generator=g), 1: torch.randn(17, 2 + 2 * hd + he, generator=g), 2: torch.randn(9, 2 + 2 * hd + he, generator=g)}
    silu = torch.nn.functional.silu

    def ref(x):
        x = silu(x.double())
        return go.decayed_memory(x[:, 2:2 + hd].reshape(-1, heads, dim), x[:, 2 + hd:2 + 2 * hd].reshape(-1, heads, dim),
                                 x[:, 2 + 2 * hd:].reshape(-1, heads, vdim), decay)[0]
    want = {i: ref(x) for i, x in full.items()}
    state = torch.full((3, heads, dim, vdim), 7.0).cuda()
    slot = {0: 2, 1: 0, 2: 2}
    cuts = {0: cuts_of(130, [1, 2, 9, 8, 1, 1, 130]), 1: cuts_of(17, [5, 1, 1, 2, 17]), 2: cuts_of(9, [2, 1, 6])}
    at = {0: 0, 1: 0, 2: 0}
    got = {i: [] for i in full}
    dec = torch.tensor(decay).cuda()
    order = [[0, 1]] * 4 + [[0]] * 10 + [[1]] * 5 + [[2, 1]] * 5
    for live in order:
        live = [i for i in live if at[i] < len(full[i]) and cuts[i]]
        if not live:
            continue
        lens = [cuts[i].pop(0) for i in live]
        x = torch.cat([full[i][at[i]:at[i] + n] for i, n in zip(live, lens)]).cuda()
        decode = all(n == 1 for n in lens) and all(at[i] > 0 for i in live)
        out = ops.decay_scan(x, (2, 2 + hd, 2 + 2 * hd), dec, state, step_layout(ops, lens, [at[i] for i in live], [slot[i] for i in live], decode),
                             heads, dim, vdim, act="silu").cpu()
        a = 0
        for i, n in zip(live, lens):
            got[i].append(out[a:a + n])
            a += n
            at[i] += n
    for i in full:
        assert at[i] == len(full[i])
        close(torch.cat(got[i]), want[i], 1e-4, f"sequence {i}")
    # the first token still counts at the end of the long sequence (heads with decay near one)
    other = ref(full[0][1:])
    assert (other[-1, 1:] - want[0][-1, 1:]).abs().max() > 1e-3


@pytest.mark.parametrize("chunk", [16, 128, None])
def test_decayed_memory_in_chunks_side_by_side(chunk):
    """Long portions are cut into chunks that run side by side, the states at their starts carried between two launches: three
    sequences of unequal length (one shorter than a chunk, one ending exactly at a chunk's edge), first from empty states, then
    continued from the states the first step left; against the walk token by token of the restatement."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(3)
    heads, dim, vdim = 3, 40, 24
    decay = [0.7, 0.99, 1.0]
    hd, he = heads * dim, heads * vdim
    n1, n2 = [600, 9, 256], [530, 700, 1]
    full = [torch.randn(a + b, 2 * hd + he, generator=g) * 0.5 for a, b in zip(n1, n2)]

    def ref(x):
        return go.decayed_memory(x[:, :hd].double().reshape(-1, heads, dim), x[:, hd:2 * hd].double().reshape(-1, heads, dim),
                                 x[:, 2 * hd:].double().reshape(-1, heads, vdim), decay)
    want = [ref(x) for x in full]
    state = torch.full((4, heads, dim, vdim), 7.0).cuda()
    dec = torch.tensor(decay).cuda()
    slots = [2, 0, 3]
    first = ops.decay_scan(torch.cat([x[:a] for x, a in zip(full, n1)]).cuda(), (0, hd, 2 * hd), dec, state,
                           step_layout(ops, n1, [0, 0, 0], slots), heads, dim, vdim, chunk=chunk).cpu()
    second = ops.decay_scan(torch.cat([x[a:] for x, a in zip(full, n1)]).cuda(), (0, hd, 2 * hd), dec, state,
                            step_layout(ops, n2, n1, slots), heads, dim, vdim, chunk=chunk).cpu()
    a1 = a2 = 0
    for b in range(3):
        close(first[a1:a1 + n1[b]], want[b][0][:n1[b]], 1e-4, f"sequence {b}, from an empty state")
        close(second[a2:a2 + n2[b]], want[b][0][n1[b]:], 1e-4, f"sequence {b}, continued")
        close(state[slots[b]].cpu(), want[b][1], 1e-4, f"sequence {b}, state left behind")
        a1, a2 = a1 + n1[b], a2 + n2[b]
    assert (state[1].cpu() == 7.0).all()


@pytest.mark.parametrize("top,experts", [(1, 3), (2, 5), (3, 3)])
def test_experts_from_a_table_by_rows_and_by_expert_order(top, experts):
    from nano_vllm_x_amd.layers.moe import TableMoE
    g = torch.Generator().manual_seed(top)
    width, ff, vocab, t = 40, 24, 19, 50
    p = {f"e{j}.{s}": torch.randn((ff, width) if s != "down" else (width, ff), generator=g) * 0.3 for j in range(experts) for s in ("gate", "up", "down")}
    p["table"] = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(vocab)]).to(torch.int32)
    moe = TableMoE(width, experts, top, ff, vocab).float().cuda()
    with torch.no_grad():
        for j in range(experts):
            moe.w_gu[j, :ff], moe.w_gu[j, ff:], moe.w_d[j] = p[f"e{j}.gate"].cuda(), p[f"e{j}.up"].cuda(), p[f"e{j}.down"].cuda()
        moe.table.copy_(p["table"])
    h = torch.randn(t, width, generator=g)
    ids = torch.randint(0, vocab, (t,), generator=g)
    want = go.table_experts(p, "", {"router": {"top": top}}, h.double(), ids)
    with torch.inference_mode():
        close(moe(h.cuda(), ids.cuda(), decode_step=False).cpu(), want, 1e-4, "expert order")          # 50 tokens: per-expert products
        close(moe(h.cuda(), ids.cuda(), decode_step=True).cpu(), want, 1e-4, "rows")                   # the decode form on the same input
        close(moe(h[:3].cuda(), ids[:3].cuda()).cpu(), want[:3], 1e-4, "few tokens")


# ---- one mixer at a time -------------------------------------------------------------------------------------------------
def _par(left=None, right=None, mlp=None, **scales):
    m = {"left": dict(LEFT, **(left or {})), "right": dict(RIGHT, **(right or {})), "left_scale": 0.7, "right_scale": 1.3}
    m.update(scales)
    return {"type": "parallel", "mixer": m, "mlp": mlp}


ONE = {
    "attention": [dict(ATT, mlp=None)],
    "attention, borrowed keys": [ATT, borrowing(ATT, 0, None), borrowing(dict(ATT, mixer=dict(ATT["mixer"], heads=2, scale=0.4)), 0, DENSE)],
    "parallel": [_par()],
    "parallel, pairs side by side": [_par(left={"rot": {"dims": 24, "base": 90.0, "layout": "interleaved"}})],
    "parallel, one head, window 1": [_par(left={"heads": 1, "kv_heads": 1, "dim": 6, "vdim": 2, "mask": {"size": 1}, "rot": {"dims": 2, "base": 10.0}},
                                          right={"heads": 1, "dim": 1, "vdim": 1, "decay": [0.8]})],
    "parallel, wide window, experts": [_par(left={"mask": {"size": 1000}, "kv_heads": 4}, mlp=MOE1, left_scale=1.0, right_scale=0.25)],
    "dense feed-forward": [dict(ATT, mlp=DENSE)],
    "experts, three of three": [dict(ATT, mlp={"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "top": 3}})],
}


@pytest.mark.parametrize("name", list(ONE))
def test_each_mixer_alone_whole_cut_and_token_by_token(tmp_path, name):
    cfg = make_cfg(ONE[name])
    w = weights_of(cfg, 1)
    eng = make_engine(model_dir(tmp_path, cfg, w), pool=256)
    toks = tokens(61, cfg["vocab"], 3)
    want = forward(cfg, w, toks)
    close(replay(eng, {"a": toks}, [[("a", 61)]])["a"], want, F32_TOL, "whole")
    close(replay(eng, {"b": toks}, [[("b", n)] for n in cuts_of(61, [2, 7, 1, 9, 3, 8, 16])])["b"], want, F32_TOL, "cut")
    close(replay(eng, {"c": toks}, [[("c", 1)]] * 61)["c"], want, F32_TOL, "token by token")
    eng.shutdown()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_fit_no_vector_width(tmp_path, dtype):
    """A width, head sizes, feed-forward sizes and a vocabulary that are multiples of nothing useful (no 16-byte rows anywhere), three
    query heads on one key/value head, experts in the first layer and a dense feed-forward in the last."""
    odd = [{"type": "attention", "mixer": {"heads": 3, "kv_heads": 1, "dim": 10, "vdim": 6, "scale": 0.3}, "mlp": {"kind": "moe", "expert": {"ff": 9}, "router": {"experts": 4, "top": 3}}},
           _par(left={"heads": 3, "kv_heads": 3, "dim": 6, "vdim": 10, "mask": {"size": 4}, "rot": {"dims": 4, "base": 77.0}, "softcap": None},
                right={"heads": 2, "dim": 5, "vdim": 7, "decay": [0.3, 0.97]}, mlp=None),
           borrowing({"mixer": {"heads": 1, "kv_heads": 1, "dim": 10, "vdim": 6, "scale": 1.0}}, 0, {"kind": "dense", "ff": 11, "limit": 0.7})]
    odd[1]["mixer"]["left"].pop("softcap")
    cfg = make_cfg(odd, width=50, vocab=37, emb=1.0, cap=0.0)
    cfg.pop("logit_softcap")
    cfg.pop("embedding")
    w = weights_of(cfg, 4)
    eng = make_engine(model_dir(tmp_path, cfg, w), dtype=dtype, pool=256)
    toks = tokens(45, 37, 8)
    want = forward(cfg, w, toks)
    got = replay(eng, {"a": toks}, [[("a", 33)], [("a", 2)]] + [[("a", 1)]] * 10)["a"]
    if dtype == "float32":
        close(got, want, F32_TOL, "float32")
        close(replay(eng, {"b": toks}, [[("b", 45)]])["b"], want, F32_TOL, "whole")
    else:
        err = (got.double() - want).abs().amax(dim=1) / want.std()
        assert err.median() < 0.08 and err.max() < 0.4, (err.median().item(), err.max().item())
    eng.shutdown()


def test_first_tokens_and_window_edges_in_prompts_and_decoding(tmp_path):
    """A window of 9 over prompts of 1, 2, 8, 9, 10 tokens and over decoded tokens that cross it one by one; key tiles of 64 crossed
    in the layers without a window; a portion that starts in the middle of a window."""
    cfg = make_cfg([PAR, ATT, PAR])
    w = weights_of(cfg, 12)
    for name in w:                               # peaked scores: a key too many or too few moves the result far
        if name.endswith(("left.q", "left.k", "mix.q", "mix.k")):
            w[name] = (w[name] * 3.0).to(torch.bfloat16).float()
    eng = make_engine(model_dir(tmp_path, cfg, w), pool=1024)
    toks = tokens(140, cfg["vocab"], 6)
    want = forward(cfg, w, toks)
    for n in (1, 2, 8, 9, 10, 64, 65):
        close(replay(eng, {f"p{n}": toks[:n]}, [[(f"p{n}", n)]])[f"p{n}"], want[:n], F32_TOL, f"prompt of {n}")
    sched = [[("a", 7)]] + [[("a", 1)]] * 5 + [[("a", 4)], [("a", 46)]] + [[("a", 1)]] * 4 + [[("a", 2)], [("a", 63)]] + [[("a", 1)]] * 9
    assert sum(n for step in sched for _, n in step) == 140
    close(replay(eng, {"a": toks}, sched)["a"], want, F32_TOL, "edges crossed token by token")
    eng.shutdown()


# ---- the whole stack ------------------------------------------------------------------------------------------------------
def test_batches_of_unequal_requests_in_a_small_pool(tmp_path):
    """Four live requests at most in a pool smaller than the sum of all: portions beside single tokens, a request that
    pauses for some steps, token slots and state slots that change hands (six requests, four state slots)."""
    cfg = make_cfg([PAR, ATT, borrowing(ATT, 1), PAR])
    w = weights_of(cfg, 2)
    eng = make_engine(model_dir(tmp_path, cfg, w), pool=160, max_bs=4)
    req = {f"r{k}": tokens(n, cfg["vocab"], 30 + k) for k, n in enumerate([70, 41, 1, 23, 55, 38])}
    want = {i: forward(cfg, w, t) for i, t in req.items()}
    sched = [[("r0", 16), ("r1", 2)], [("r0", 1), ("r1", 30), ("r2", 1)], [("r0", 40), ("r3", 3)], [("r1", 1), ("r3", 1)],
             [("r0", 1), ("r1", 1), ("r3", 17)], [("r0", 12), ("r1", 7), ("r3", 2)],          # r0, r1, r3 done: 134 slots come back
             [("r4", 2), ("r5", 30)], [("r4", 50), ("r5", 1)], [("r4", 1), ("r5", 1)], [("r4", 2), ("r5", 6)]]
    got = replay(eng, req, sched)
    for i in req:
        close(got[i], want[i], F32_TOL, i)
    assert eng.scheduler.state_slots.num_free() == 4
    eng.shutdown()


def test_far_tokens_and_old_state_count(tmp_path):
    cfg = make_cfg([_par(right={"decay": [0.999, 0.9, 1.0]}, mlp=MOE2), ATT, borrowing(ATT, 1), PAR])
    w = weights_of(cfg, 7)
    for name in w:
        if name.endswith(("mix.q", "mix.k")):
            w[name] = (w[name] * 3.0).to(torch.bfloat16).float()
        if name.endswith(".r1"):
            w[name] = w[name] * 0.1              # a weak distance penalty: the far keys keep their weight
    eng = make_engine(model_dir(tmp_path, cfg, w), pool=512)
    toks = tokens(330, cfg["vocab"], 2)
    want = forward(cfg, w, toks)
    got = replay(eng, {"a": toks}, [[("a", 255)], [("a", 1)], [("a", 1)], [("a", 2)], [("a", 30)]] + [[("a", 1)]] * 41)["a"]
    close(got, want, F32_TOL, "sharpened")
    # the same prompt without its first token is another function of the rest: the first token is seen at the end
    other = forward(cfg, w, toks[1:])
    assert (other[-1] - want[-1]).abs().max() > 20 * F32_TOL * want.std()
    eng.shutdown()


def test_bfloat16_stays_within_rounding(tmp_path):
    cfg = make_cfg([PAR, ATT, borrowing(ATT, 1)])
    toks = tokens(90, cfg["vocab"], 4)
    want = forward(cfg, weights_of(cfg, 2), toks)
    eng = make_engine(model_dir(tmp_path, cfg), dtype="bfloat16", seed=2)
    got = replay(eng, {"a": toks}, [[("a", 50)], [("a", 2)]] + [[("a", 1)]] * 38)["a"]
    err = (got.double() - want).abs().amax(dim=1) / want.std()
    assert err.median() < 0.08 and err.max() < 0.4, (err.median().item(), err.max().item())
    eng.shutdown()


def test_checkpoint_with_a_missing_or_misshapen_tensor_is_refused(tmp_path):
    cfg = make_cfg([PAR, ATT])
    w = weights_of(cfg, 0)
    bad = dict(w)
    del bad["l0.mix.right.norm"]
    with pytest.raises(KeyError):
        make_engine(model_dir(tmp_path, cfg, bad, name="missing"))
    bad = dict(w)
    bad["l0.mix.left.v"] = torch.zeros(41, cfg["width"])
    with pytest.raises(ValueError):
        make_engine(model_dir(tmp_path, cfg, bad, name="shape"))
    bad = dict(w)
    bad["l0.mlp.table"] = torch.full_like(w["l0.mlp.table"], 5)
    with pytest.raises(ValueError):
        make_engine(model_dir(tmp_path, cfg, bad, name="table"))


# ---- generation: the scheduler's own choices ---------------------------------------------------------------------------
def oracle_greedy(w, cfg, prompt, n_new):
    return greedy(lambda t: forward(cfg, w, t), prompt, n_new)


@pytest.mark.parametrize("chunked", [False, True], ids=["whole prompts", "chunked prefill"])
def test_greedy_generation_through_the_engine(tmp_path, chunked):
    """Prompts of unequal length admitted together, decoded as one batch; more requests than state slots, so the later ones wait
    for a slot that an earlier one gives back; with chunked prefill the prompts are computed in portions of seven tokens.  Long
    decoding (30 tokens, past the window) for one of them."""
    from nano_vllm_x_amd.core.common import SamplingParams
    cfg = make_cfg([PAR, ATT, borrowing(ATT, 1)])
    kw = dict(max_prefill_tokens=7, chunked_prefill=True) if chunked else {}
    eng = make_engine(model_dir(tmp_path, cfg), pool=300, max_bs=3, seed=9, **kw)
    w = weights_of(cfg, 9)
    prompts = {f"r{k}": tokens(n, cfg["vocab"], 20 + k) for k, n in enumerate([5, 19, 1, 12, 9])}
    new = {"r0": 30, "r1": 5, "r2": 8, "r3": 4, "r4": 6}
    for i, p in prompts.items():
        eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=new[i]))
    out = {i: [] for i in prompts}
    steps = 0
    while eng.has_unfinished_sequences():
        for o in eng.step():
            out[o.seq_id].append(o.new_token_id)
        steps += 1
        assert steps < 400
    for i, p in prompts.items():
        assert out[i] == oracle_greedy(w, cfg, p, new[i]), i
    assert eng.scheduler.state_slots.num_free() == 3
    eng.shutdown()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replay_a_captured_graph(tmp_path, dtype):
    """With graphs on, every decode step replays the graph of its batch size, with prefill steps of later requests (eager work on
    the same cache and state) between the replays; batch sizes change as requests end.  float32: the tokens are the
    restatement's; bfloat16: the graph's tokens are those of eager steps (same kernels, same order)."""
    from nano_vllm_x_amd.core.common import SamplingParams
    from nano_vllm_x_amd.core.engine import Engine
    cfg = make_cfg([PAR, ATT, borrowing(ATT, 1), _par(mlp=DENSE)])
    path = model_dir(tmp_path, cfg)
    prompts = {f"r{k}": tokens(n, cfg["vocab"], 40 + k) for k, n in enumerate([9, 26, 2, 17, 5])}
    new = {"r0": 20, "r1": 5, "r2": 11, "r3": 3, "r4": 7}

    def run(eager):
        eng = Engine(model=path, gpu_memory_utilization=0.5, max_bs=3, enforce_eager=eager, context_len=128, kv_cache_size=300,
                     dtype=dtype, seed=5)
        for i, p in prompts.items():
            eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=new[i]))
        out = {i: [] for i in prompts}
        while eng.has_unfinished_sequences():
            for o in eng.step():
                out[o.seq_id].append(o.new_token_id)
        stats = dict(eng.model_runner.stats)
        eng.shutdown()
        return out, stats

    got, stats = run(False)
    assert stats["graph_steps"] > 15 and stats["eager_decode_steps"] == 0
    if dtype == "float32":
        w = weights_of(cfg, 5)
        for i, p in prompts.items():
            assert got[i] == oracle_greedy(w, cfg, p, new[i]), i
    else:
        assert got == run(True)[0]


def test_generate_entry_point(tmp_path):
    from nano_vllm_x_amd import LLM, SamplingParams
    cfg = make_cfg([ATT, PAR], vocab=300)
    llm = LLM(model_dir(tmp_path, cfg), gpu_memory_utilization=0.5, max_bs=2, enforce_eager=True, context_len=256, kv_cache_size=256,
              dtype="float32", seed=4)
    prompt = tokens(11, 300, 1)

    async def run():
        ids = []
        async for o in llm.generate(list(prompt), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=5, eos_token_id=0)):
            ids.append(o.token_id)
        return ids

    assert asyncio.run(run()) == oracle_greedy(weights_of(cfg, 4), cfg, prompt, 5)
    llm.shutdown()


def test_preempted_sequence_starts_again_from_an_empty_state(tmp_path):
    from nano_vllm_x_amd.core.common import SamplingParams
    cfg = make_cfg([PAR, ATT])
    eng = make_engine(model_dir(tmp_path, cfg), pool=64, max_bs=2, seed=6)
    w = weights_of(cfg, 6)
    prompts = {"a": tokens(20, cfg["vocab"], 1), "b": tokens(25, cfg["vocab"], 2)}
    for i, p in prompts.items():
        eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=14))
    out = {i: [] for i in prompts}
    while eng.has_unfinished_sequences():       # 45 + 2 * 14 tokens do not fit 64 slots: the younger sequence is preempted
        for o in eng.step():
            out[o.seq_id].append(o.new_token_id)
    for i, p in prompts.items():
        assert out[i] == oracle_greedy(w, cfg, p, 14), i
    eng.shutdown()


def test_command_line_generates_what_the_restatement_does(tmp_path):
    import subprocess
    import sys
    cfg = make_cfg([ATT, PAR], vocab=90)
    path = model_dir(tmp_path, cfg)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-m", "nano_vllm_x_amd", "--model", path, "--prompt-ids", "5,17,3,44", "--prompt-ids", "8",
                          "--max-new-tokens", "6", "--dtype", "float32", "--kv-cache-size", "128", "--context-len", "64", "--max-bs", "2",
                          "--seed", "3"], cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [json.loads(x) for x in out.stdout.splitlines() if x.startswith("{")]
    w = weights_of(cfg, 3)
    assert [x["prompt"] for x in lines] == [[5, 17, 3, 44], [8]]
    for x in lines:
        assert x["generated_ids"] == oracle_greedy(w, cfg, x["prompt"], 6)


def test_trace_runner_replays_steps_from_standard_input(tmp_path):
    """bin/trace_run on a model directory: two requests, portions beside single tokens, one request ended and its id used again;
    the logits it writes are the restatement's."""
    import subprocess
    cfg = make_cfg([PAR, ATT], vocab=80)
    w = weights_of(cfg, 11)
    path = model_dir(tmp_path, cfg, w)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = tokens(30, 80, 1), tokens(12, 80, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}, {"id": "b", "tokens": b[:1], "want": [0]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[9:29], "want": []}, {"id": "b", "tokens": b[1:], "want": [10]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[29:], "want": [0]}, {"id": "b", "tokens": a[:5], "want": [4]}], "end": ["a", "b"]}]
    out_dir = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(out_dir), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.splitlines() if x.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = forward(cfg, w, a), forward(cfg, w, b)
    got = [torch.from_numpy(np.fromfile(out_dir / f"{k}.f32", dtype="<f4").reshape(-1, 80).copy()) for k in range(3)]
    close(got[0], torch.stack([la[0], la[8], lb[0]]), F32_TOL, "step 0")
    close(got[1], lb[11:12], F32_TOL, "step 1")
    close(got[2], torch.stack([la[29], la[4]]), F32_TOL, "step 2")
