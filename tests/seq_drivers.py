"""Drivers shared by the GPU tests of models with per-sequence state: model directories, engines, replay of given steps,
ragged step layouts, comparison against a restatement."""
import json

import numpy as np
import torch

F32_TOL = 2e-4


def model_dir(tmp_path, cfg, weights=None, name="m"):
    """A directory as a user's: config.json and, if `weights` are given, model.safetensors (bfloat16; integer tables as int32)."""
    d = tmp_path / name
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    if weights is not None:
        from safetensors.torch import save_file
        save_file({k: (v.to(torch.int32) if not v.is_floating_point() else v.to(torch.bfloat16)).contiguous() for k, v in weights.items()},
                  str(d / "model.safetensors"))
    return str(d)


def make_engine(path, dtype="float32", pool=2048, max_bs=4, seed=0, **kw):
    from nano_vllm_x_amd.core.engine import Engine
    return Engine(model=path, gpu_memory_utilization=0.5, max_bs=max_bs, enforce_eager=True, context_len=pool, kv_cache_size=pool,
                  dtype=dtype, seed=seed, **kw)


def replay(engine, requests, schedule):
    """requests: id -> tokens; schedule: list of steps, each a list of (id, n).  Logits of every token, id -> (T, vocab)."""
    from nano_vllm_x_amd.core.common import SamplingParams
    at = {i: 0 for i in requests}
    rows = {i: [] for i in requests}
    for step in schedule:
        plan, want = [], []
        for i, n in step:
            piece = list(requests[i][at[i]:at[i] + n])
            if engine.scheduler.get_sequence(i) is None:
                engine.add_sequence(i, piece, SamplingParams(ignore_eos=True))
            else:
                engine.extend_sequence(i, piece)
            plan.append((i, n))
            want.append(list(range(n)))
        out = engine.run_given(plan, want).float().cpu()
        k = 0
        for i, n in step:
            rows[i].append(out[k:k + n])
            k += n
            at[i] += n
            if at[i] == len(requests[i]):
                engine.abort_sequence(i)
    return {i: torch.cat(r) for i, r in rows.items()}


def close(got, want, tol, what=""):
    got, want = got.double(), want.double()
    scale = want.std().item() + 1e-12
    err = (got - want).abs().max().item() / scale
    assert err < tol, f"{what}: max error {err:.3e} of the values' spread (tolerance {tol})"


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def cuts_of(n, sizes):
    """n tokens cut into portions whose sizes cycle through `sizes`."""
    out, k = [], 0
    while n > 0:
        c = min(sizes[k % len(sizes)], n)
        out.append(c)
        n -= c
        k += 1
    return out


def step_layout(ops, lens, pos0, slots, decode=False):
    """ops.StepLayout of a step that brings lens[b] tokens of sequence b from position pos0[b], its state in slots[b]."""
    n = len(lens)
    p, s = torch.tensor(pos0, dtype=torch.int64).cuda(), torch.tensor(slots, dtype=torch.int32).cuda()
    if decode:
        return ops.StepLayout(n, n, p, s)
    qo = np.zeros(n + 1, dtype=np.int32)
    np.cumsum(lens, out=qo[1:])
    tok = np.repeat(np.arange(n, dtype=np.int32), lens)
    return ops.StepLayout(int(qo[-1]), n, p, s, torch.from_numpy(qo).cuda(), torch.from_numpy(tok).cuda())


def greedy(forward, prompt, n_new):
    """n_new tokens by arg-max of `forward(tokens)[-1]`, recomputing the whole sequence each time."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(toks)[-1].argmax()))
    return toks[len(prompt):]
