"""Papunex family on the CPU path: every mechanism against the plain
oracle (tests/papunex_oracle.py), then the engine — scheduler, paged
latent cache, recurrent state rows — against whole-sequence oracle
logits under prefill, decode, chunking, batching and page/row reuse."""

from __future__ import annotations

import math
import random

import pytest
import torch

from tests import papunex_oracle as O
from tests.gadilix_harness import chunked, run_schedule, whole

TOL = 3e-4   # fp32 end to end, relative to the largest logit


def _tokens(n, vocab, seed):
    rnd = random.Random(seed)
    return [rnd.randrange(vocab) for _ in range(n)]


def _close(got, ref, tol=TOL):
    err = (got.float() - ref.float()).abs().max().item()
    assert err <= tol * max(1.0, ref.abs().max().item()), err


def _model(tmp_path_factory, name, layers, seed, **kw):
    cfg = O.make_config(layers, **kw)
    wt = O.random_weights(cfg, seed=seed)
    path = O.save_model(str(tmp_path_factory.mktemp(name)), cfg, wt)
    return path, cfg, wt


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    """Every branch: own keys, borrowed keys, partial rotation, both
    mixers, dense / routed / no feed-forward, with and without a shared
    expert, groups < heads, one and several norm groups."""
    layers = [
        O.latent_entry(heads=3, dim=8, rot_dim=6, vdim=4, kv_rank=12,
                       rot_dims=4, mlp="dense", ff=20),
        O.mamba_entry(heads=4, vdim=6, state=5, groups=2, conv=3,
                      norm_groups=3, mlp="moe", ff=8, experts=5, top=2,
                      router_scale=1.7, shared_ff=12),
        O.latent_entry(heads=2, dim=4, rot_dim=6, vdim=10, kv_rank=12,
                       rot_dims=4, kv_from=0, mlp=None),
        O.mamba_entry(heads=2, vdim=20, state=18, groups=1, conv=5,
                      norm_groups=1, mlp="moe", ff=8, experts=3, top=3,
                      shared_ff=0),
        O.latent_entry(heads=1, dim=16, rot_dim=2, vdim=8, kv_rank=6,
                       mlp="moe", ff=12, experts=4, top=1, shared_ff=4),
    ]
    return _model(tmp_path_factory, "papunex_a", layers, 1, vocab=40,
                  width=24, embed_scale=3.0, softcap=15.0)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    """Values that tend to be equal or 1 elsewhere are not here: one
    tap (no conv tail), groups == heads, top == experts == 1, rotation
    of nothing (dims 0), no softcap, scale 1 embedding."""
    layers = [
        O.mamba_entry(heads=3, vdim=4, state=3, groups=3, conv=1,
                      norm_groups=1, mlp=None),
        O.latent_entry(heads=2, dim=6, rot_dim=2, vdim=6, kv_rank=5,
                       rot_dims=0, mlp="moe", ff=8, experts=1, top=1,
                       shared_ff=8),
        O.mamba_entry(heads=1, vdim=40, state=20, groups=1, conv=2,
                      norm_groups=4, mlp="dense", ff=8),
    ]
    return _model(tmp_path_factory, "papunex_b", layers, 2, vocab=33,
                  width=20, embed_scale=1.0, softcap=0.0)


# ---------------------------------------------------------------------
# Mechanisms alone (ops of the CPU path vs the oracle).

def test_weighted_norm_and_residual_update():
    from vllm_amd import ops

    y = torch.randn(5, 24)
    w = torch.rand(24) + 0.5
    ref = O.rms(y, 1e-3) * w
    _close(ops.rms_norm_cast(y, w, 1e-3, torch.float32), ref, 1e-6)
    x = torch.randn(5, 24)
    want = x + ref
    copy = ops.add_rms_norm(x, y, w, 1e-3, torch.bfloat16)
    _close(x, want, 1e-6)
    assert copy.dtype == torch.bfloat16
    assert ops.add_rms_norm(x, y, w, 1e-3) is x


def test_small_elementwise_ops():
    from vllm_amd import ops

    x = torch.randn(7, 10) * 3
    _close(ops.relu2(x), torch.relu(x) ** 2, 1e-6)
    _close(ops.logit_softcap(x * 20, 11.0), 11.0 * torch.tanh(x * 20 / 11.0),
           1e-6)
    table = torch.randn(9, 6)
    ids = torch.tensor([3, 0, 8, 3])
    _close(ops.scaled_embedding(ids, table, 2.5), table[ids] * 2.5, 1e-6)
    h = torch.randn(4, 3, 5)
    g = torch.randn(4, 15)
    got = ops.sigmoid_gate_mul(h.transpose(0, 1).contiguous()
                               .transpose(0, 1), g)
    _close(got, h.reshape(4, 15) * torch.sigmoid(g), 1e-6)


def test_router_scores_renormalise_and_scale():
    from vllm_amd import ops

    z = torch.randn(6, 7) * 2
    w, ids = ops.softmax_topk_scaled(z, 3, 1.9)
    s = torch.softmax(z, -1)
    for t in range(6):
        order = sorted(range(7), key=lambda e: -float(s[t, e]))[:3]
        assert sorted(ids[t].tolist()) == sorted(order)
        tot = sum(float(s[t, e]) for e in order)
        for k in range(3):
            assert abs(float(w[t, k])
                       - float(s[t, ids[t, k]]) / tot * 1.9) < 1e-6


def test_squared_relu_experts_ungated():
    from vllm_amd import ops

    torch.manual_seed(0)
    E, ff, width, T = 4, 6, 10, 9
    up = torch.randn(E, ff, width)
    down = torch.randn(E, width, ff)
    x = torch.randn(T, width)
    w = torch.rand(T, 2)
    ids = torch.stack([torch.randperm(E)[:2] for _ in range(T)]).int()
    got = ops.fused_moe(x, up, down, w, ids, activation="relu2")
    ref = torch.zeros(T, width)
    for t in range(T):
        for k in range(2):
            e = int(ids[t, k])
            ref[t] += w[t, k] * O.relu2_mlp(x[t:t + 1], up[e], down[e])[0]
    _close(got, ref, 1e-5)


def _latent_through_cache(q_abs, q_rot, rows, scale, sink, cuts, bs=16,
                          device="cpu", dtype=torch.float32):
    """Feed one sequence through the paged attention op in portions;
    rows [T, L+R] are written as they are (already normed/rotated)."""
    from vllm_amd import ops

    T = q_abs.shape[0]
    nb = -(-T // bs) + 3
    cache = torch.full((nb, bs, rows.shape[1]), 5.0, dtype=dtype,
                       device=device)
    pages = list(range(nb))
    random.Random(3).shuffle(pages)
    bt = torch.tensor([pages], dtype=torch.int32, device=device)
    outs, at = [], 0
    for n in cuts:
        n = min(n, T - at)
        if n <= 0:
            break
        pos = torch.arange(at, at + n)
        slot = bt[0].cpu()[pos // bs].long() * bs + pos % bs
        cache.view(-1, rows.shape[1])[slot.to(device)] = \
            rows[at:at + n].to(device, dtype)
        qsl = torch.tensor([0, n], dtype=torch.int32, device=device)
        sl = torch.tensor([at + n], dtype=torch.int32, device=device)
        outs.append(ops.latent_attention(
            q_abs[at:at + n].to(device, dtype),
            q_rot[at:at + n].to(device, dtype), cache, bt, qsl, sl, scale,
            sink=None if sink is None else sink.to(device),
            num_decodes=1 if n == 1 else 0, max_seq_len=at + n,
            max_query_len=n).float().cpu())
        at += n
    return torch.cat(outs)


def _latent_plain(q_abs, q_rot, rows, scale, sink):
    T, H, L = q_abs.shape
    out = torch.zeros(T, H, L)
    for t in range(T):
        for h in range(H):
            s = (rows[:t + 1, :L] @ q_abs[t, h]
                 + rows[:t + 1, L:] @ q_rot[t, h]) * scale
            sk = -math.inf if sink is None else float(sink[h])
            m = max(float(s.max()), sk)
            e = torch.exp(s - m)
            den = e.sum() + (0.0 if sink is None else math.exp(sk - m))
            out[t, h] = (e[:, None] * rows[:t + 1, :L]).sum(0) / den
    return out


@pytest.mark.parametrize("L,R,use_sink", [(6, 4, True), (9, 2, False),
                                          (5, 0, True)])
def test_latent_attention_op_cuts_and_pages(L, R, use_sink):
    torch.manual_seed(L * 10 + R)
    T, H = 70, 3
    q_abs = torch.randn(T, H, L)
    q_rot = torch.randn(T, H, R)
    rows = torch.randn(T, L + R)
    sink = torch.randn(H) if use_sink else None
    ref = _latent_plain(q_abs, q_rot, rows, 0.4, sink)
    for cuts in ([T], [1] * T, [2, 14, 1, 1, 15, 17, 2, 100]):
        _close(_latent_through_cache(q_abs, q_rot, rows, 0.4, sink, cuts),
               ref, 1e-5)


def test_sink_takes_weight_but_gives_nothing():
    """A towering sink leaves (almost) nothing for the keys; a very low
    one changes nothing."""
    T, H, L = 20, 2, 4
    q_abs = torch.randn(T, H, L)
    q_rot = torch.zeros(T, H, 2)
    rows = torch.randn(T, L + 2)
    none = _latent_through_cache(q_abs, q_rot, rows, 1.0, None, [T])
    low = _latent_through_cache(q_abs, q_rot, rows, 1.0,
                                torch.full((H,), -60.0), [7, 13])
    high = _latent_through_cache(q_abs, q_rot, rows, 1.0,
                                 torch.tensor([40.0, -60.0]), [T])
    _close(low, none, 1e-6)
    assert high[:, 0].abs().max() < 1e-6
    _close(high[:, 1], none[:, 1], 1e-6)


@pytest.mark.parametrize("far", [0, 15, 16, 63, 64, 200])
def test_single_far_key_dominates(far):
    """All latent rows are small except one far back (at and next to
    page borders) whose score towers: every later position returns that
    row, earlier ones do not see it."""
    T, L = 330, 4
    rows = torch.zeros(T, L + 2)
    rows[:, 0] = 0.01
    rows[far, :L] = torch.tensor([3.0, -2.0, 1.0, 4.0])
    q_abs = torch.zeros(T, 1, L)
    q_abs[:, 0, 3] = 20.0
    q_rot = torch.zeros(T, 1, 2)
    for cuts in ([T], [far + 1] + [1] * 40 + [T], [64, 64, 64, 3, 200]):
        out = _latent_through_cache(q_abs, q_rot, rows, 1.0, None, cuts)
        for t in (far, far + 1, T - 1):
            _close(out[t, 0], rows[far, :L], 1e-5)
        if far:
            assert out[far - 1, 0, 3].abs() < 1e-6


def test_rotation_and_cache_write():
    from vllm_amd import ops
    from vllm_amd.layers.rotary import PairwiseRotary

    torch.manual_seed(5)
    T, H, D, R, L, dims = 6, 2, 3, 6, 5, 4
    rot = PairwiseRotary(dims, 50.0)
    q = torch.randn(T, H, D + R)
    dkv = torch.randn(T, L + R)
    w = torch.rand(L) + 0.5
    pos = torch.tensor([0, 1, 7, 64, 65, 1000])
    cache = torch.zeros(3, 4, L + R)
    slots = torch.tensor([5, 0, 11, 2, -1, 7])
    q_ref = q.clone()
    ops.latent_rope_cache_write(q, dkv, w, 1e-4, pos, rot.inv_freq, D, L,
                                cache, slots)
    flat = cache.view(-1, L + R)
    for t in range(T):
        p = int(pos[t])
        for h in range(H):
            _close(q[t, h, :D], q_ref[t, h, :D], 0)
            _close(q[t, h, D:], O.rotate_pairs(q_ref[t, h, D:], p, 50.0,
                                               dims), 1e-5)
        if slots[t] < 0:
            continue
        _close(flat[slots[t], :L], O.rms(dkv[t, :L], 1e-4) * w, 1e-5)
        _close(flat[slots[t], L:], O.rotate_pairs(dkv[t, L:], p, 50.0,
                                                  dims), 1e-5)
    assert flat[1].abs().sum() == 0          # untouched slot


@pytest.mark.parametrize("K", [1, 2, 4, 7])
def test_conv_carries_its_tail_across_chunks(K):
    from vllm_amd import ops

    torch.manual_seed(K)
    T, C = 23, 6
    x = torch.randn(T, C)
    w = torch.randn(C, K)
    b = torch.randn(C)
    ref = O.causal_conv_silu(x, w, b)
    for cuts in ([T], [1] * T, [2, 1, 5, 1, 1, 9, 4]):
        state = torch.randn(3, C, K - 1)
        state[2] = 0
        rows = torch.tensor([2])
        outs, at = [], 0
        for n in cuts:
            qsl = torch.tensor([0, n], dtype=torch.int32)
            outs.append(ops.causal_conv_silu(x[at:at + n], w, b, state,
                                             rows, qsl))
            at += n
        _close(torch.cat(outs), ref, 1e-5)
        if K > 1:
            _close(state[2], x[T - (K - 1):].t(), 0)


def test_scan_carries_state_and_batches():
    from vllm_amd import ops

    torch.manual_seed(9)
    Hm, P, G, N = 4, 5, 2, 3
    lens = [9, 1, 14]
    seqs = []
    for n in lens:
        seqs.append((torch.randn(n, Hm * P + 2 * G * N),
                     torch.randn(n, Hm)))
    dt_bias, a_log = torch.randn(Hm) - 1, torch.randn(Hm) * 0.5
    d_skip = torch.randn(Hm)
    refs = []
    for xbc, dt in seqs:
        n = xbc.shape[0]
        refs.append(O.ssd_scan(
            xbc[:, :Hm * P].reshape(n, Hm, P),
            xbc[:, Hm * P:Hm * P + G * N].reshape(n, G, N),
            xbc[:, Hm * P + G * N:].reshape(n, G, N),
            torch.nn.functional.softplus(dt + dt_bias), torch.exp(a_log),
            d_skip, G))
    # Three requests side by side, in two steps, rows 4, 0, 2.
    state = torch.zeros(5, Hm, P, N)
    rows = torch.tensor([4, 0, 2])
    got = [[], [], []]
    for lo, hi in ((0, 0.4), (0.4, 1.0)):
        parts, qsl = [], [0]
        for j, (xbc, dt) in enumerate(seqs):
            n = xbc.shape[0]
            a, b = (int(n * lo), int(n * hi)) if n > 1 else \
                ((0, 1) if lo == 0 else (1, 1))
            parts.append((xbc[a:b], dt[a:b]))
            qsl.append(qsl[-1] + b - a)
        y = ops.ssd_scan(torch.cat([p[0] for p in parts]), Hm, P, G, N,
                         torch.cat([p[1] for p in parts]), dt_bias, a_log,
                         d_skip, state, rows,
                         torch.tensor(qsl, dtype=torch.int32))
        for j in range(3):
            got[j].append(y[qsl[j]:qsl[j + 1]])
    for j in range(3):
        _close(torch.cat(got[j]), refs[j], 1e-5)
    assert state[1].abs().sum() == 0 and state[3].abs().sum() == 0


def test_gate_comes_before_the_group_norm():
    from vllm_amd import ops

    y = torch.randn(4, 12)
    z = torch.randn(4, 12)
    w = torch.rand(12) + 0.5
    g = y * (z * torch.sigmoid(z))
    ref = O.rms(g.view(4, 3, 4), 1e-3).reshape(4, 12) * w
    _close(ops.gated_group_rms_norm(y, z, w, 1e-3, 3, torch.float32), ref,
           1e-6)


# ---------------------------------------------------------------------
# The engine against the oracle.

def _ref(model, tokens):
    _, cfg, wt = model
    return O.forward(cfg, wt, tokens)


def _check(got, rid, ref, positions=None):
    for p in (range(ref.shape[0]) if positions is None else positions):
        _close(got[(rid, p)], ref[p])


@pytest.mark.parametrize("which", ["a", "b"])
def test_whole_prompt_and_layers(which, model_a, model_b):
    model = model_a if which == "a" else model_b
    toks = _tokens(90, model[1]["vocab"], 11)
    ref = _ref(model, toks)
    got, _ = run_schedule(model[0], whole("r", toks), max_tokens=128)
    _check(got, "r", ref)


def test_residual_stream_after_every_layer(model_a):
    from vllm_amd.entrypoints.trace_replay import build_core, replay
    import json
    import tempfile

    path, cfg, wt = model_a
    toks = _tokens(21, cfg["vocab"], 3)
    _, layers = O.forward(cfg, wt, toks, return_layers=True)
    core = build_core(path, "float32", 64, "cpu")
    seen = {}
    core.worker.runner.model.model.layer_probe = \
        lambda i, x: seen.__setitem__(i, x.clone())
    try:
        replay(core, [json.dumps({"step": 0, "entries": [
            {"id": "r", "tokens": toks, "want": []}], "end": ["r"]})],
            tempfile.mkdtemp(), lambda s: None)
    finally:
        core.shutdown()
    for i in range(len(cfg["layers"])):
        _close(seen[i], layers[i], 1e-4)


@pytest.mark.parametrize("which", ["a", "b"])
def test_prefill_against_token_by_token(which, model_a, model_b):
    model = model_a if which == "a" else model_b
    toks = _tokens(75, model[1]["vocab"], 5)
    ref = _ref(model, toks)
    got, _ = run_schedule(model[0], chunked("r", toks, [1] * 75),
                          max_tokens=128)
    _check(got, "r", ref)
    got, _ = run_schedule(model[0], chunked("r", toks, [40] + [1] * 35),
                          max_tokens=128)
    _check(got, "r", ref)


@pytest.mark.parametrize("sizes", [[2] * 40, [3, 2, 61, 2, 5, 1, 1, 2],
                                   [63, 1, 1, 2], [64, 2, 64], [7] * 20])
def test_portions(sizes, model_a):
    toks = _tokens(131, model_a[1]["vocab"], 7)
    ref = _ref(model_a, toks)
    got, _ = run_schedule(model_a[0], chunked("r", toks, sizes),
                          max_tokens=192)
    _check(got, "r", ref)


def test_unequal_batch_against_each_alone(model_a):
    vocab = model_a[1]["vocab"]
    reqs = {"a": _tokens(70, vocab, 1), "b": _tokens(9, vocab, 2),
            "c": _tokens(130, vocab, 3), "d": _tokens(1, vocab, 4)}
    refs = {k: _ref(model_a, v) for k, v in reqs.items()}
    at = {k: 0 for k in reqs}
    plan = [{"a": 30, "b": 1, "c": 2}, {"a": 1, "c": 64, "d": 1},
            {"a": 1, "b": 3, "c": 1}, {"b": 5, "c": 63}, {"a": 38},
            {"c": 0}]
    steps = []
    for st in plan:
        ent, end = [], []
        for k, n in st.items():
            n = min(n, len(reqs[k]) - at[k]) if n else len(reqs[k]) - at[k]
            ent.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        steps.append((ent, end))
    assert all(at[k] == len(reqs[k]) for k in reqs)
    got, _ = run_schedule(model_a[0], steps, max_tokens=448)
    for k in reqs:
        _check(got, k, refs[k])


def test_pages_and_rows_are_reused(model_a):
    """Ten requests through four rows and a pool that holds two of
    them at a time; later ones land on pages and rows that earlier ones
    left full of their keys and state."""
    vocab = model_a[1]["vocab"]
    steps, refs = [], {}
    for i in range(10):
        toks = _tokens(50 + 7 * (i % 3), vocab, 20 + i)
        refs[f"r{i}"] = (toks, _ref(model_a, toks))
    names = list(refs)
    for i in range(0, 10, 2):
        a, b = names[i], names[i + 1]
        ta, tb = refs[a][0], refs[b][0]
        steps.append(([(a, ta[:20], list(range(20))), (b, tb[:1], [0])], []))
        steps.append(([(a, ta[20:], list(range(len(ta) - 20))),
                       (b, tb[1:], list(range(len(tb) - 1)))], [a, b]))
    got, _ = run_schedule(model_a[0], steps, max_tokens=128)
    for k, (_, ref) in refs.items():
        _check(got, k, ref)


def test_first_tokens_and_one_token_prompt(model_b):
    vocab = model_b[1]["vocab"]
    for n in (1, 2, 3):
        toks = _tokens(n, vocab, 30 + n)
        got, _ = run_schedule(model_b[0], whole("r", toks), max_tokens=64)
        _check(got, "r", _ref(model_b, toks))


def test_long_decode(model_b):
    toks = _tokens(260, model_b[1]["vocab"], 8)
    ref = _ref(model_b, toks)
    got, _ = run_schedule(model_b[0], chunked("r", toks, [5] + [1] * 255),
                          max_tokens=320)
    _check(got, "r", ref, positions=range(0, 260, 7))
    _check(got, "r", ref, positions=[63, 64, 65, 127, 128, 129, 255, 259])


def test_bad_configs_are_rejected(tmp_path):
    from vllm_amd.config import get_model_spec

    def spec(layers):
        cfg = O.make_config(layers)
        return get_model_spec(O.save_model(
            str(tmp_path / f"m{random.random()}"), cfg, {}))

    with pytest.raises(ValueError):
        spec([O.latent_entry(kv_from=0)])
    with pytest.raises(ValueError):
        spec([O.mamba_entry(), O.latent_entry(kv_from=0)])
    with pytest.raises(ValueError):
        spec([O.latent_entry(kv_rank=8),
              O.latent_entry(kv_rank=6, kv_from=0)])
    bad = O.latent_entry()
    bad["type"] = "something"
    with pytest.raises(ValueError):
        spec([bad])


def test_greedy_generation_through_llm(model_a):
    """LLM.generate -> scheduler -> runner -> sampler: each greedy token
    is the oracle's argmax given the tokens so far."""
    from vllm_amd.entrypoints.llm import LLM
    from vllm_amd.sampling_params import SamplingParams

    path, cfg, wt = model_a
    prompts = [_tokens(12, cfg["vocab"], 40), _tokens(3, cfg["vocab"], 41)]
    llm = LLM(model=path, model_path=path, load_format="safetensors",
              dtype="fp32", device="cpu", num_gpu_blocks=8,
              max_model_len=128, max_num_seqs=4, max_num_batched_tokens=8)
    try:
        outs = llm.generate(
            prompts, SamplingParams(temperature=0.0, max_tokens=6,
                                    ignore_eos=True))
    finally:
        llm.shutdown()
    for p, o in zip(prompts, outs):
        gen = list(o.outputs[0].token_ids)
        assert len(gen) == 6
        seq = list(p)
        for tok in gen:
            logits = O.forward(cfg, wt, seq)[-1]
            top2 = logits.topk(2).values
            if float(top2[0] - top2[1]) > 1e-3:
                assert tok == int(logits.argmax())
            seq.append(tok)


def test_served_over_http(model_a):
    """The OpenAI-compatible server loads the folder like any other
    model; token-id prompt, greedy completion, the oracle's tokens (the
    family has no tokenizer: ids come back as text bytes)."""
    from fastapi.testclient import TestClient

    from vllm_amd.engine.arg_utils import EngineArgs
    from vllm_amd.entrypoints.openai.api_server import make_server

    path, cfg, wt = model_a
    prompt = _tokens(9, cfg["vocab"], 77)
    seq = list(prompt)
    sure = True
    for _ in range(4):
        logits = O.forward(cfg, wt, seq)[-1]
        top2 = logits.topk(2).values
        sure = sure and float(top2[0] - top2[1]) > 1e-3
        seq.append(int(logits.argmax()))
    args = EngineArgs(model=path, model_path=path, load_format="safetensors",
                      dtype="fp32", device="cpu", num_gpu_blocks=8,
                      max_model_len=256, max_num_seqs=4,
                      max_num_batched_tokens=64)
    app, state = make_server(args, None)
    try:
        with TestClient(app) as c:
            r = c.post("/v1/completions", json={
                "model": path, "prompt": prompt, "max_tokens": 4,
                "temperature": 0})
            assert r.status_code == 200, r.text
    finally:
        state.engine.shutdown()
    text = r.json()["choices"][0]["text"]
    assert len(text) == 4
    if sure:
        assert [ord(ch) for ch in text] == seq[len(prompt):]
