"""Gadilix family on the MI355X path: HIP kernels (row-wise and MFMA
pooled-window attention, fused q/k norm + cache write, pooled-block
finalize, fp32 residual ops) and the engine on the GPU against the
plain oracle (tests/gadilix_oracle.py)."""

from __future__ import annotations

import random

import pytest
import torch

from tests import gadilix_oracle as O
from tests.gadilix_harness import (attention_through_cache, chunked,
                                   run_schedule, whole)

pytestmark = pytest.mark.gpu


def _tokens(n, vocab, seed):
    rnd = random.Random(seed)
    return [rnd.randrange(vocab) for _ in range(n)]


def _close(got, ref, tol):
    err = (got.float().cpu() - ref).abs().max().item()
    assert err <= tol * max(1.0, ref.abs().max().item()), err


def _round(t, dtype):
    return t.to(dtype).float()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5),
                                       (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,D,Dv,Wn,P", [
    (6, 3, 56, 40, 44, 11), (8, 2, 64, 32, 17, 5), (4, 1, 36, 72, 33, 64),
    (4, 4, 128, 128, 100, 1), (2, 2, 256, 200, 7, 100), (3, 1, 20, 12, 1, 3),
    (10, 2, 32, 48, 300, 7),
])
def test_attention_kernels(dtype, tol, H, G, D, Dv, Wn, P):
    torch.manual_seed(H * 1000 + D)
    T = 330
    q = _round(torch.randn(T, H, D) * 1.5, dtype)
    k = _round(torch.randn(T, G, D), dtype)
    v = _round(torch.randn(T, G, Dv), dtype)
    scale = 2.0 / D ** 0.5
    ref = O.pooled_window_attention(q, k, v, scale, Wn, P)
    for cuts in ([T], [200] + [1] * 130, [2, 61, 1, 1, 3, 64, 2, 130, 66]):
        got = attention_through_cache(q, k, v, scale, Wn, P, cuts,
                                      device="cuda", dtype=dtype)
        _close(got, ref, tol)


def _oracle_rows(q, k, v, scale, Wn, P, rows):
    """The oracle's attention for a few positions of one sequence."""
    H, G = q.shape[1], k.shape[1]
    out = torch.zeros(len(rows), H, v.shape[2])
    for n, i in enumerate(rows):
        toks, blocks = O.visible_keys(i, Wn, P)
        for g in range(G):
            K = torch.stack([k[j, g] for j in toks]
                            + [k[b * P:b * P + P, g].mean(0) for b in blocks])
            V = torch.stack([v[j, g] for j in toks]
                            + [v[b * P:b * P + P, g].mean(0) for b in blocks])
            for h in range(g * (H // G), (g + 1) * (H // G)):
                w = torch.softmax((K @ q[i, h]) * scale, dim=0)
                out[n, h] = w @ V
    return out


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2),
                                       (torch.float16, 4e-3),
                                       (torch.float32, 2e-5)])
@pytest.mark.parametrize("H,G,D,Dv,Wn,P", [
    (10, 2, 64, 128, 128, 16), (8, 1, 128, 64, 600, 64), (3, 3, 40, 24, 9, 2),
])
def test_batched_decode_rows(dtype, tol, H, G, D, Dv, Wn, P):
    """Several decode rows of unequal context in one launch, with the
    output gate, beside a prompt chunk in the same batch; every row
    against the oracle on its own sequence."""
    from vllm_amd import ops

    torch.manual_seed(H + Wn)
    bs = 64
    lens = [1, 5, 64, 65, 300, 700, Wn, Wn + P, Wn + P + 1]
    chunk = 37                       # prompt chunk after the decode rows
    n_dec = len(lens)
    lens_all = lens + [chunk + 90]
    pages_per = [-(-n // bs) for n in lens_all]
    nb = sum(pages_per) + 2
    order = list(range(nb))
    random.Random(5).shuffle(order)
    slots = ops.pool_slots_per_page(P, bs)
    kc = torch.zeros(nb, G, bs, D, dtype=dtype, device="cuda")
    vc = torch.zeros(nb, G, bs, Dv, dtype=dtype, device="cuda")
    pk = torch.zeros(nb, G, slots, D, device="cuda")
    pv = torch.zeros(nb, G, slots, Dv, device="cuda")
    bt = torch.zeros(len(lens_all), max(pages_per), dtype=torch.int32)
    at = 0
    for r, n in enumerate(pages_per):
        bt[r, :n] = torch.tensor(order[at:at + n], dtype=torch.int32)
        at += n
    bt = bt.cuda()
    seqs = []
    for r, L in enumerate(lens_all):
        q = _round(torch.randn(L, H, D) * 1.5, dtype)
        k = _round(torch.randn(L, G, D), dtype)
        v = _round(torch.randn(L, G, Dv), dtype)
        gate = _round(torch.randn(L, H), dtype)
        seqs.append((q, k, v, gate))
        # Everything before this step's tokens goes in as one chunk.
        new = 1 if r < n_dec else chunk
        old = L - new
        if old:
            pos = torch.arange(old)
            slot = (bt[r, pos // bs].cpu().long() * bs + pos % bs).cuda()
            ops.norm_qk_cache_write(
                q[:old].to("cuda", dtype), k[:old].to("cuda", dtype),
                v[:old].to("cuda", dtype), None, None, 0.0, kc, vc, slot)
            ops.pool_update(
                kc, vc, pk, pv, bt[r:r + 1],
                torch.tensor([0, old], dtype=torch.int32, device="cuda"),
                torch.tensor([old], dtype=torch.int32, device="cuda"), P,
                max_query_len=old)
    scale = 2.0 / D ** 0.5
    news = [1] * n_dec + [chunk]
    qsl = torch.tensor([0] + list(torch.tensor(news).cumsum(0)),
                       dtype=torch.int32, device="cuda")
    sl = torch.tensor(lens_all, dtype=torch.int32, device="cuda")
    cat = lambda i: torch.cat([s[i][-n:] for s, n in zip(seqs, news)])
    pos = torch.cat([torch.arange(L - n, L) for L, n in zip(lens_all, news)])
    req = torch.cat([torch.full((n,), r) for r, n in enumerate(news)])
    slot = (bt.cpu()[req, pos // bs].long() * bs + pos % bs).cuda()
    qq = ops.norm_qk_cache_write(
        cat(0).to("cuda", dtype), cat(1).to("cuda", dtype),
        cat(2).to("cuda", dtype), None, None, 0.0, kc, vc, slot)
    ops.pool_update(kc, vc, pk, pv, bt, qsl, sl, P, max_query_len=chunk)
    out = ops.pooled_window_attention(
        qq, kc, vc, pk, pv, bt, qsl, sl, scale, Wn, P,
        gate=cat(3).to("cuda", dtype), num_decodes=n_dec,
        max_seq_len=max(lens_all), max_query_len=chunk).float().cpu()
    at = 0
    for (q, k, v, gate), n in zip(seqs, news):
        L = q.shape[0]
        ref = _oracle_rows(q, k, v, scale, Wn, P, range(L - n, L))
        ref = ref * torch.sigmoid(gate[-n:]).unsqueeze(-1)
        _close(out[at:at + n], ref, tol)
        at += n


def test_far_key_on_gpu_bf16():
    T, Wn, P = 700, 10, 4
    q = torch.zeros(T, 1, 16)
    k = torch.zeros(T, 1, 16)
    v = torch.zeros(T, 1, 16)
    q[:, 0, 0] = 40.0
    far = 22
    k[far, 0, 0] = 4.0
    v[:, 0, :] = (torch.arange(T).float() % 64).unsqueeze(1)
    for cuts in ([T], [300] + [1] * 400):
        out = attention_through_cache(q, k, v, 1.0, Wn, P, cuts,
                                      device="cuda", dtype=torch.bfloat16)
        assert abs(out[far + Wn - 1, 0, 0] - v[far, 0, 0]) < 0.2
        for i in (23 + Wn, 200, 450, T - 1):
            assert abs(out[i, 0, 0] - v[20:24, 0, 0].mean()) < 0.2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
# Widths on the 4-wide kernels (one and several chunks per thread), an
# odd width and one too wide for them (both on the scalar kernels).
@pytest.mark.parametrize("W", [352, 2560, 355, 4100])
def test_elementwise_kernels(dtype, W):
    from vllm_amd.ops import hip_ops as Hp

    torch.manual_seed(0)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    T = 37
    y = _round(torch.randn(T, W), dtype)
    g = torch.tensor(0.7)
    _close(Hp.scalar_rms_norm(y.to("cuda", dtype), g.cuda(), 1e-5,
                              torch.float32), O.scalar_norm(y, g, 1e-5),
           1e-5)
    x = torch.randn(T, W)
    xg = x.clone().cuda()
    copy = Hp.add_scaled_scalar_norm(xg, y.to("cuda", dtype), g.cuda(),
                                     1e-5, 0.45, dtype)
    want = x + 0.45 * O.scalar_norm(y, g, 1e-5)
    _close(xg, want, 1e-5)
    _close(copy, want, tol)
    # token shift over a batch of three requests (one empty), with carry
    mu = torch.rand(W)
    state = torch.randn(5, W)
    qsl = torch.tensor([0, 1, 1, 20, 37], dtype=torch.int32)
    rows = torch.tensor([3, 0, 4, 1])
    sg = state.clone().cuda()
    got = Hp.token_shift(x.cuda(), mu.cuda(), sg, rows.cuda(), qsl.cuda(),
                         dtype)
    for r, (s, e) in enumerate(((0, 1), (1, 1), (1, 20), (20, 37))):
        if s == e:
            continue
        seq = torch.cat([state[rows[r]][None], x[s:e]])
        _close(got[s:e], x[s:e] + (seq[:-1] - x[s:e]) * mu, tol)
        _close(sg[rows[r]], x[e - 1], 0)
    _close(sg[2], state[2], 0)
    # q/k head norm fused with the cache write
    # 8-aligned head widths take the 16 B kernel (two chunks at 136);
    # the others the scalar one.
    H, G, D, Dv, bs = {352: (4, 2, 24, 40, 64), 2560: (5, 5, 136, 256, 64),
                       355: (4, 2, 20, 40, 64),
                       4100: (18, 1, 64, 8, 64)}[W]
    q = _round(torch.randn(T, H, D), dtype)
    k = _round(torch.randn(T, G, D), dtype)
    v = _round(torch.randn(T, G, Dv), dtype)
    qw = _round(torch.rand(D) + .5, dtype)
    kw = _round(torch.rand(D) + .5, dtype)
    kc = torch.zeros(3, G, bs, D, dtype=dtype, device="cuda")
    vc = torch.zeros(3, G, bs, Dv, dtype=dtype, device="cuda")
    slot = torch.arange(T) + 70
    slot[5] = -1
    qn = Hp.norm_qk_cache_write(
        q.to("cuda", dtype), k.to("cuda", dtype), v.to("cuda", dtype),
        qw.to("cuda", dtype), kw.to("cuda", dtype), 1e-5, kc, vc,
        slot.cuda())
    _close(qn, O.unit_rms(q, 1e-5) * qw, tol)
    kn = O.unit_rms(k, 1e-5) * kw
    for t in (0, 4, 6, T - 1):
        s = int(slot[t])
        _close(kc[s // bs, :, s % bs], kn[t], tol)
        _close(vc[s // bs, :, s % bs], v[t], 0)
    assert float(kc[0].abs().max()) == 0.0


@pytest.fixture(scope="module")
def model_g(tmp_path_factory):
    layers = [
        O.layer_entry(heads=4, kv_heads=2, dim=48, vdim=40, window=20,
                      pool=6, ff=32, shared_ff=64),
        O.layer_entry(heads=2, kv_heads=1, dim=64, vdim=64, window=70,
                      pool=3, mlp=False),
        O.layer_entry(heads=4, kv_heads=2, dim=48, vdim=40, window=20,
                      pool=6, ff=32, shared_ff=64, weights_of=0),
        O.layer_entry(heads=3, kv_heads=3, dim=16, vdim=24, window=5,
                      pool=66, experts=3, top=1, ff=16, shared_ff=16),
    ]
    cfg = O.make_config(layers, vocab=96, width=64, residual_mult=0.4)
    wt = O.random_weights(cfg, seed=2, sharp=2.0)
    path = O.save_model(str(tmp_path_factory.mktemp("gadilix_g")), cfg, wt)
    return path, cfg, wt


def _mixed_steps(reqs):
    at = {r: 0 for r in reqs}

    def take(r, n):
        n = min(n, len(reqs[r]) - at[r])
        ent = (r, reqs[r][at[r]:at[r] + n], list(range(n)))
        at[r] += n
        return ent

    steps = [
        ([take("a", 60), take("b", 2), take("c", 9)], ["c"]),
        ([take("a", 1), take("b", 47), take("d", 5)], []),
        ([take("a", 1), take("b", 1), take("d", 1), take("g", 3)],
         ["b", "g"]),
        ([take("a", 68), take("d", 64), take("e", 30), take("f", 2)],
         ["a", "d"]),
        ([take("e", 1), take("f", 1)], []),
        ([take("e", 69), take("f", 61)], ["e", "f"]),
    ]
    assert all(at[r] == len(reqs[r]) for r in reqs)
    return steps


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-4),
                                       ("bfloat16", 0.15)])
def test_engine_on_gpu(model_g, dtype, tol):
    path, cfg, wt = model_g
    V = cfg["vocab"]
    toks = _tokens(230, V, 1)
    ref = O.forward(cfg, wt, toks)
    for steps in (whole("a", toks),
                  chunked("a", toks, [150] + [1] * 80),
                  chunked("a", toks, [2, 61, 1, 1, 3, 64, 2, 70, 2])):
        got, _ = run_schedule(path, steps, dtype=dtype, device="cuda")
        for p in range(len(toks)):
            _close(got[("a", p)], ref[p], tol)
    reqs = {r: _tokens(n, V, 20 + i) for i, (r, n) in enumerate(
        [("a", 130), ("b", 50), ("c", 9), ("d", 70), ("e", 100),
         ("f", 64), ("g", 3)])}
    got, core = run_schedule(path, _mixed_steps(reqs), dtype=dtype,
                             max_tokens=7 * 64, device="cuda")
    for r, t in reqs.items():
        ref = O.forward(cfg, wt, t)
        for p in range(len(t)):
            _close(got[(r, p)], ref[p], tol)


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-4),
                                       ("bfloat16", 0.15)])
def test_unaligned_sizes_on_gpu(tmp_path, dtype, tol):
    """Width, vocab, head and expert widths that are multiples of
    neither 8 nor 16: the scalar kernels and the unaligned GEMM route."""
    layers = [
        O.layer_entry(heads=5, kv_heads=1, dim=24, vdim=40, window=9,
                      pool=4, experts=5, top=2, ff=28, shared_ff=36),
        O.layer_entry(heads=2, kv_heads=2, dim=20, vdim=12, window=33,
                      pool=64, experts=2, top=2, ff=10, shared_ff=6),
        O.layer_entry(heads=6, kv_heads=2, dim=8, vdim=8, window=64,
                      pool=1, mlp=False),
    ]
    cfg = O.make_config(layers, vocab=101, width=100, residual_mult=0.7)
    wt = O.random_weights(cfg, seed=9, sharp=2.0)
    path = O.save_model(str(tmp_path / "m"), cfg, wt)
    toks = _tokens(140, 101, 6)
    ref = O.forward(cfg, wt, toks)
    got, _ = run_schedule(path, chunked("a", toks, [3, 70, 2] + [1] * 65),
                          dtype=dtype, device="cuda")
    for p in range(len(toks)):
        _close(got[("a", p)], ref[p], tol)


def test_grouped_gemm_expert_path(tmp_path):
    """Widths that qualify for the grouped-GEMM MFMA expert kernels
    (width % 128 == 0, ff % 64 == 0, bf16)."""
    layers = [O.layer_entry(heads=4, kv_heads=4, dim=64, vdim=64,
                            window=30, pool=8, experts=6, top=2, ff=64,
                            shared_ff=128)] * 2
    cfg = O.make_config(layers, vocab=80, width=256, residual_mult=0.35)
    wt = O.random_weights(cfg, seed=3, sharp=2.0)
    path = O.save_model(str(tmp_path / "m"), cfg, wt)
    toks = _tokens(150, 80, 4)
    ref = O.forward(cfg, wt, toks)
    got, _ = run_schedule(path, chunked("a", toks, [100] + [1] * 50),
                          dtype="bfloat16", device="cuda")
    for p in range(len(toks)):
        _close(got[("a", p)], ref[p], 0.15)


def test_captured_decode_matches_eager(tmp_path):
    """One-token steps replayed from captured hipGraphs (batch buckets
    with padded rows, requests joining and leaving, state rows staged
    per step) against the eager engine and the oracle."""
    layers = [O.layer_entry(heads=4, kv_heads=2, dim=64, vdim=32,
                            window=30, pool=8, experts=6, top=2, ff=64,
                            shared_ff=128),
              O.layer_entry(heads=4, kv_heads=2, dim=64, vdim=32,
                            window=30, pool=8, experts=6, top=2, ff=64,
                            shared_ff=128, weights_of=0),
              O.layer_entry(heads=8, kv_heads=1, dim=32, vdim=64,
                            window=300, pool=5, mlp=False)]
    cfg = O.make_config(layers, vocab=80, width=256, residual_mult=0.35)
    wt = O.random_weights(cfg, seed=5, sharp=2.0)
    path = O.save_model(str(tmp_path / "m"), cfg, wt)
    reqs = {"a": _tokens(150, 80, 41), "b": _tokens(90, 80, 42),
            "c": _tokens(70, 80, 43)}
    steps = [([("a", reqs["a"][:100], [99]), ("b", reqs["b"][:50], [49])],
              [])]
    for i in range(40):                       # two decode rows
        steps.append(([("a", reqs["a"][100 + i:101 + i], [0]),
                       ("b", reqs["b"][50 + i:51 + i], [0])],
                      ["b"] if i == 39 else []))
    steps.append(([("c", reqs["c"][:60], [59])], []))
    for i in range(10):                       # other rows, other bucket
        steps.append(([("a", reqs["a"][140 + i:141 + i], [0]),
                       ("c", reqs["c"][60 + i:61 + i], [0])],
                      ["a", "c"] if i == 9 else []))
    graph, core = run_schedule(path, steps, dtype="bfloat16",
                               device="cuda", enforce_eager=False)
    assert core.worker.runner.graph_runner is not None
    assert core.worker.runner.graph_runner.graphs, "nothing was captured"
    eager, _ = run_schedule(path, steps, dtype="bfloat16", device="cuda")
    assert graph.keys() == eager.keys()
    for r, t in reqs.items():
        ref = O.forward(cfg, wt, t)
        for (rid, p_), got in graph.items():
            if rid != r:
                continue
            _close(got, eager[(rid, p_)], 2e-2)
            _close(got, ref[p_], 0.15)


def test_greedy_generation_on_gpu(model_g):
    from vllm_amd.entrypoints.llm import LLM
    from vllm_amd.sampling_params import SamplingParams

    path, cfg, wt = model_g
    prompts = [_tokens(37, cfg["vocab"], 31), _tokens(5, cfg["vocab"], 32)]
    n_new = 10
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(n_new):
            seq.append(int(O.forward(cfg, wt, seq)[-1].argmax()))
        want.append(seq[len(p):])
    llm = LLM(model=path, model_path=path, load_format="safetensors",
              dtype="fp32", device="cuda", num_gpu_blocks=8,
              max_model_len=128, max_num_seqs=4, max_num_batched_tokens=16)
    try:
        outs = llm.generate(
            prompts, SamplingParams(temperature=0.0, max_tokens=n_new,
                                    ignore_eos=True))
    finally:
        llm.shutdown()
    assert [list(o.outputs[0].token_ids) for o in outs] == want
