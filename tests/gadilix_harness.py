"""Drive the engine with a step schedule and collect tapped logits."""

from __future__ import annotations

import json
import os
import tempfile

import random

import numpy as np
import torch


def run_schedule(model_dir, steps, dtype="float32", max_tokens=1024,
                 device="cpu", enforce_eager=True):
    """steps: list of (entries, end) with entries = [(req_id, tokens,
    want_offsets)]. Returns {(req_id, absolute position): logits}."""
    from vllm_amd.entrypoints.trace_replay import build_core, replay

    lines, wanted, seen = [], [], {}
    for n, (entries, end) in enumerate(steps):
        row = []
        ent = []
        for rid, toks, want in entries:
            base = seen.get(rid, 0)
            ent.append({"id": rid, "tokens": list(toks),
                        "want": list(want)})
            row += [(rid, base + w) for w in want]
            seen[rid] = base + len(toks)
        for rid in end:
            seen.pop(rid, None)
        lines.append(json.dumps({"step": n, "entries": ent,
                                 "end": list(end)}))
        wanted.append(row)
    out = tempfile.mkdtemp()
    core = build_core(model_dir, dtype, max_tokens, device,
                      enforce_eager=enforce_eager)
    done = []
    try:
        replay(core, lines, out, done.append)
    finally:
        core.shutdown()
    assert done == [f"done {n}" for n in range(len(steps))]
    got = {}
    for n, row in enumerate(wanted):
        path = os.path.join(out, f"{n}.f32")
        if not row:
            assert not os.path.exists(path)
            continue
        arr = np.fromfile(path, dtype="<f4").reshape(len(row), -1)
        for j, key in enumerate(row):
            got[key] = torch.from_numpy(arr[j].copy())
    return got, core


def whole(rid, tokens, want=None):
    want = list(range(len(tokens))) if want is None else want
    return [([(rid, tokens, want)], [rid])]


def chunked(rid, tokens, sizes):
    """One request alone, cut into the given portion sizes (the last
    portion takes what is left); every position is wanted."""
    steps, at = [], 0
    sizes = list(sizes)
    while at < len(tokens):
        n = sizes.pop(0) if sizes else len(tokens) - at
        n = min(n, len(tokens) - at)
        steps.append(([(rid, tokens[at:at + n], list(range(n)))], []))
        at += n
    steps[-1] = (steps[-1][0], [rid])
    return steps


def attention_through_cache(q, k, v, scale, Wn, P, cuts, bs=64,
                             device="cpu", dtype=torch.float32,
                             shuffle_pages=True):
    """Feed one sequence through the paged ops in the given portions."""
    from vllm_amd import ops

    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    nb = -(-T // bs) + 3
    slots = ops.pool_slots_per_page(P, bs)
    kc = torch.full((nb, G, bs, D), 7.0, dtype=dtype, device=device)
    vc = torch.full((nb, G, bs, Dv), -7.0, dtype=dtype, device=device)
    pk = torch.full((nb, G, slots, D), 9.0, device=device)
    pv = torch.full((nb, G, slots, Dv), -9.0, device=device)
    pages = list(range(nb))
    if shuffle_pages:
        random.Random(3).shuffle(pages)
    bt = torch.tensor([pages], dtype=torch.int32, device=device)
    outs, at = [], 0
    for n in cuts:
        n = min(n, T - at)
        if n <= 0:
            break
        pos = torch.arange(at, at + n)
        slot = (bt[0, pos // bs].cpu().long() * bs + pos % bs).to(device)
        qsl = torch.tensor([0, n], dtype=torch.int32, device=device)
        sl = torch.tensor([at + n], dtype=torch.int32, device=device)
        qq = ops.norm_qk_cache_write(
            q[at:at + n].to(device, dtype), k[at:at + n].to(device, dtype),
            v[at:at + n].to(device, dtype), None, None, 0.0, kc, vc, slot)
        ops.pool_update(kc, vc, pk, pv, bt, qsl, sl, P, max_query_len=n)
        outs.append(ops.pooled_window_attention(
            qq, kc, vc, pk, pv, bt, qsl, sl, scale, Wn, P,
            num_decodes=1 if n == 1 else 0, max_seq_len=at + n,
            max_query_len=n).float().cpu())
        at += n
    return torch.cat(outs)
