"""Gadilix family on the CPU path: every mechanism against the plain
oracle (tests/gadilix_oracle.py), then the engine — scheduler, paged
cache, pooled areas, shift-carry rows — against whole-sequence oracle
logits under prefill, decode, chunking, batching and page/row reuse."""

from __future__ import annotations

import math
import random

import pytest
import torch

from tests import gadilix_oracle as O
from tests.gadilix_harness import (attention_through_cache as
                                   _attention_through_cache, chunked,
                                   run_schedule, whole)

TOL = 2e-4   # fp32 end to end; logits are O(1)


def _tokens(n, vocab, seed):
    rnd = random.Random(seed)
    return [rnd.randrange(vocab) for _ in range(n)]


def _close(got, ref, tol=TOL):
    err = (got - ref).abs().max().item()
    assert err <= tol * max(1.0, ref.abs().max().item()), err


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    """GQA, key width != value width, a layer without feed-forward, a
    layer that borrows weights, different windows/pools per layer."""
    layers = [
        O.layer_entry(heads=4, kv_heads=2, dim=8, vdim=12, window=6,
                      pool=3),
        O.layer_entry(heads=2, kv_heads=1, dim=16, vdim=8, window=9,
                      pool=4, mlp=False),
        O.layer_entry(heads=4, kv_heads=2, dim=8, vdim=12, window=6,
                      pool=3, weights_of=0),
        O.layer_entry(heads=3, kv_heads=3, dim=8, vdim=8, window=5,
                      pool=7, experts=3, top=1, ff=8, shared_ff=8),
    ]
    cfg = O.make_config(layers, vocab=40, width=32, residual_mult=0.4)
    wt = O.random_weights(cfg, seed=1)
    path = O.save_model(str(tmp_path_factory.mktemp("gadilix_a")), cfg, wt)
    return path, cfg, wt


# ---------------------------------------------------------------------
# Mechanisms alone (torch reference ops of the CPU path vs the oracle).

def test_scalar_norm_and_residual_update():
    from vllm_amd import ops

    y = torch.randn(5, 24)
    g = torch.tensor(0.7)
    ref = O.scalar_norm(y, g, 1e-3)
    _close(ops.scalar_rms_norm(y, g, 1e-3), ref, 1e-6)
    x = torch.randn(5, 24)
    want = x + 0.45 * ref
    copy = ops.add_scaled_scalar_norm(x, y, g, 1e-3, 0.45, torch.bfloat16)
    _close(x, want, 1e-6)
    assert copy.dtype == torch.bfloat16


def test_token_shift_carries_across_chunks():
    from vllm_amd import ops

    h = torch.randn(11, 16)
    mu = torch.rand(16)
    ref = O.token_shift(h, mu)
    state = torch.randn(3, 16)
    state[1] = 0                       # fresh row
    rows = torch.tensor([1])
    outs = []
    for s, e in ((0, 4), (4, 5), (5, 7), (7, 11)):
        qsl = torch.tensor([0, e - s], dtype=torch.int32)
        outs.append(ops.token_shift(h[s:e].clone(), mu, state, rows, qsl,
                                    torch.float32))
    _close(torch.cat(outs), ref, 1e-6)
    _close(state[1], h[-1], 0)


@pytest.mark.parametrize("P,bs", [(1, 64), (3, 64), (12, 64), (64, 64),
                                  (100, 64), (5, 16)])
def test_pool_slot_layout_is_collision_free(P, bs):
    """Every pooled block gets its own (page, slot) and fits the page's
    slot count."""
    from vllm_amd.ops._torch_ref import _pool_slot, pool_slots_per_page

    slots = pool_slots_per_page(P, bs)
    seen = set()
    for b in range(0, 2000 // P + 2):
        page, slot = _pool_slot(b, P, bs)
        assert 0 <= slot < slots
        assert page == (b * P + P - 1) // bs
        assert (page, slot) not in seen
        seen.add((page, slot))


def _visible(i, Wn, P):
    return O.visible_keys(i, Wn, P)


def test_visibility_rule_edges():
    # window 4, blocks of 3: position 9 sees tokens 6..9; block 1
    # (3..5) ends at 5 = 9 - 4: just seen; at position 8 it is not yet
    # (and tokens 3, 4 are then seen by nobody).
    assert _visible(9, 4, 3) == ([6, 7, 8, 9], [0, 1])
    assert _visible(8, 4, 3) == ([5, 6, 7, 8], [0])
    assert _visible(2, 4, 3) == ([0, 1, 2], [])
    assert _visible(6, 4, 3) == ([3, 4, 5, 6], [0])
    assert _visible(5, 4, 3) == ([2, 3, 4, 5], [])


@pytest.mark.parametrize("Wn,P", [(6, 3), (44, 11), (1, 1), (5, 70),
                                  (64, 64), (65, 2), (200, 5)])
def test_pooled_window_attention_op(Wn, P):
    torch.manual_seed(Wn * 100 + P)
    T, H, G, D, Dv = 150, 4, 2, 8, 12
    q = torch.randn(T, H, D) * 2
    k = torch.randn(T, G, D)
    v = torch.randn(T, G, Dv)
    ref = O.pooled_window_attention(q, k, v, 0.5, Wn, P)
    for cuts in ([T], [1] * T, [2, 61, 1, 1, 3, 64, 2, 100]):
        _close(_attention_through_cache(q, k, v, 0.5, Wn, P, cuts), ref,
               1e-5)


def test_single_far_key_dominates():
    """All keys are zero except one far back whose score towers over
    the rest: the output is (almost) that key's pooled block mean once
    the block is seen, and before that the key is invisible."""
    T, Wn, P = 300, 10, 4
    q = torch.zeros(T, 1, 4)
    k = torch.zeros(T, 1, 4)
    v = torch.zeros(T, 1, 4)
    q[:, 0, 0] = 50.0
    far = 22                              # block 5 = positions 20..23
    k[far, 0, 0] = 4.0                    # pooled mean -> 1.0, score 50
    v[:, 0, :] = torch.arange(T).float().unsqueeze(1)
    for cuts in ([T], [7] * 50, [1] * T):
        out = _attention_through_cache(q, k, v, 1.0, Wn, P, cuts)
        blk_mean = v[20:24, 0, 0].mean()
        # in the window: the key itself wins
        assert abs(out[far + Wn - 1, 0, 0] - far) < 1e-3
        # block ends at 23: seen from position 23 + Wn on
        first_seen = 23 + Wn
        # left the window, block not yet seen: every visible score is
        # zero, so the output is the plain average of what is visible
        for i in range(far + Wn, first_seen):
            toks, blocks = O.visible_keys(i, Wn, P)
            assert far not in toks and 5 not in blocks
            vals = [float(j) for j in toks] + [
                float(v[b * P:b * P + P, 0, 0].mean()) for b in blocks]
            assert abs(out[i, 0, 0] - sum(vals) / len(vals)) < 1e-3
        for i in (first_seen, first_seen + 1, 150, T - 1):
            assert abs(out[i, 0, 0] - blk_mean) < 1e-3, (i, out[i, 0, 0])


def test_output_gate_scales_each_head():
    """The gate multiplies head h of token t by sigmoid(gate[t, h]); a
    very negative gate silences one head and leaves the others."""
    torch.manual_seed(4)
    from vllm_amd import ops
    T, H, G, D, Dv, Wn, P, bs = 70, 4, 2, 8, 6, 9, 4, 64
    q, k, v = torch.randn(T, H, D), torch.randn(T, G, D), \
        torch.randn(T, G, Dv)
    gate = torch.randn(T, H)
    gate[:, 2] = -40.0
    ref = O.pooled_window_attention(q, k, v, 0.4, Wn, P) \
        * torch.sigmoid(gate).unsqueeze(-1)
    kc, vc = torch.zeros(3, G, bs, D), torch.zeros(3, G, bs, Dv)
    slots = ops.pool_slots_per_page(P, bs)
    pk, pv = torch.zeros(3, G, slots, D), torch.zeros(3, G, slots, Dv)
    bt = torch.tensor([[2, 0, 1]], dtype=torch.int32)
    pos = torch.arange(T)
    slot = bt[0, pos // bs].long() * bs + pos % bs
    qsl = torch.tensor([0, T], dtype=torch.int32)
    sl = torch.tensor([T], dtype=torch.int32)
    qq = ops.norm_qk_cache_write(q, k, v, None, None, 0.0, kc, vc, slot)
    ops.pool_update(kc, vc, pk, pv, bt, qsl, sl, P, max_query_len=T)
    out = ops.pooled_window_attention(qq, kc, vc, pk, pv, bt, qsl, sl, 0.4,
                                      Wn, P, gate=gate, max_seq_len=T,
                                      max_query_len=T)
    _close(out, ref, 1e-5)
    assert float(out[:, 2].abs().max()) < 1e-12


def test_table_routed_experts_alone():
    """The feed-forward module by itself: experts come from the token
    id's table row with weight 1/top each, plus the shared expert; the
    activations play no part in the choice."""
    from vllm_amd.models.gadilix import GadilixMoE

    torch.manual_seed(6)
    V, W = 23, 16
    for experts, top, shared in ((5, 2, 12), (3, 3, None), (4, 1, 8)):
        ml = {"kind": "moe", "expert": {"ff": 10},
              "router": {"experts": experts, "top": top}}
        if shared:
            ml["shared"] = {"ff": shared}
        cfg = O.make_config([dict(O.layer_entry(), mlp=ml)], vocab=V,
                            width=W)
        wt = O.random_weights(cfg, seed=experts)
        moe = GadilixMoE(W, V, ml, torch.float32)
        moe.router.table.copy_(wt["l0.mlp.table"])
        moe.experts.load_full_weights(
            torch.stack([wt[f"l0.mlp.e{e}.gate"] for e in range(experts)]),
            torch.stack([wt[f"l0.mlp.e{e}.up"] for e in range(experts)]),
            torch.stack([wt[f"l0.mlp.e{e}.down"] for e in range(experts)]))
        if shared:
            moe.shared.gate_up_proj.weight.data.copy_(torch.cat(
                [wt["l0.mlp.shared.gate"], wt["l0.mlp.shared.up"]]))
            moe.shared.down_proj.weight.data.copy_(
                wt["l0.mlp.shared.down"])
        toks = torch.tensor([0, 22, 7, 7, 13, 1, 0])
        x = torch.randn(len(toks), W)
        want = O.table_moe(x, toks.tolist(), wt, "l0.mlp.", ml)
        _close(moe(x, toks), want, 1e-5)
        # Same token id, other activations: same experts.
        x2 = torch.randn(len(toks), W) * 30
        _close(moe(x2, toks), O.table_moe(x2, toks.tolist(), wt,
                                          "l0.mlp.", ml), 1e-4)


# ---------------------------------------------------------------------
# The engine against whole-sequence oracle logits.

def test_whole_prompt_logits(model_a):
    path, cfg, wt = model_a
    toks = _tokens(90, cfg["vocab"], 0)
    ref = O.forward(cfg, wt, toks)
    got, _ = run_schedule(path, whole("a", toks))
    for p in range(len(toks)):
        _close(got[("a", p)], ref[p])


def test_first_tokens_and_single_token_prompt(model_a):
    path, cfg, wt = model_a
    for n in (1, 2, 3):
        toks = _tokens(n, cfg["vocab"], 10 + n)
        ref = O.forward(cfg, wt, toks)
        got, _ = run_schedule(path, whole("a", toks))
        for p in range(n):
            _close(got[("a", p)], ref[p])


@pytest.mark.parametrize("sizes", [
    [1] * 70,                       # pure token-by-token decoding
    [40] + [1] * 30,                # prefill, then decode past windows
    [2, 2, 3, 5, 2, 17, 1, 1, 2, 30, 2],
    [63, 1, 1, 2],                  # page border inside portions
    [64, 6],
    [65, 5],
])
def test_portions_match_whole(model_a, sizes):
    path, cfg, wt = model_a
    toks = _tokens(70, cfg["vocab"], 5)
    ref = O.forward(cfg, wt, toks)
    got, _ = run_schedule(path, chunked("a", toks, sizes))
    for p in range(len(toks)):
        _close(got[("a", p)], ref[p])


def test_long_decoding_over_several_pages(model_a):
    path, cfg, wt = model_a
    toks = _tokens(200, cfg["vocab"], 6)
    ref = O.forward(cfg, wt, toks)
    got, _ = run_schedule(path, chunked("a", toks, [10] + [1] * 190))
    for p in range(len(toks)):
        _close(got[("a", p)], ref[p])


def test_mixed_batches_and_reuse_of_pages_and_rows(model_a):
    """Unequal requests in one batch — portions beside single tokens —
    in a pool that only fits the live ones, so finished requests' pages
    and state rows are handed to later requests."""
    path, cfg, wt = model_a
    V = cfg["vocab"]
    reqs = {r: _tokens(n, V, 20 + i) for i, (r, n) in enumerate(
        [("a", 130), ("b", 50), ("c", 9), ("d", 70), ("e", 100),
         ("f", 64), ("g", 3)])}
    refs = {r: O.forward(cfg, wt, t) for r, t in reqs.items()}
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
    # The pool is exactly the most the live requests ever hold, each
    # rounded up to pages (step 3: 3 + 2 + 1 + 1 pages).
    got, core = run_schedule(path, steps, max_tokens=7 * 64)
    pool = core.scheduler.kv_cache_manager.block_pool
    assert pool.get_num_free_blocks() == pool.num_gpu_blocks
    for r, toks in reqs.items():
        for p in range(len(toks)):
            _close(got[(r, p)], refs[r][p])


def test_other_sizes_and_degenerate_constants(tmp_path):
    """Sizes the first model does not have: one kv head, one expert,
    top = experts, pool > page, pool 1, window 1, no shared expert, odd
    widths."""
    layers = [
        O.layer_entry(heads=2, kv_heads=1, dim=6, vdim=10, window=1,
                      pool=1, experts=1, top=1, ff=4, shared_ff=12),
        O.layer_entry(heads=1, kv_heads=1, dim=24, vdim=4, window=3,
                      pool=70, experts=3, top=3, ff=12, shared_ff=4),
        O.layer_entry(heads=6, kv_heads=3, dim=4, vdim=4, window=80,
                      pool=2, experts=5, top=2, ff=20, shared_ff=8),
    ]
    layers[2]["mlp"]["shared"] = None
    cfg = O.make_config(layers, vocab=23, width=20, eps=1e-3,
                        residual_mult=1.0)
    wt = O.random_weights(cfg, seed=4)
    path = O.save_model(str(tmp_path / "m"), cfg, wt)
    toks = _tokens(160, cfg["vocab"], 8)
    ref = O.forward(cfg, wt, toks)
    got, _ = run_schedule(path, chunked("a", toks, [75, 2, 1, 1, 60] + [1] * 30))
    for p in range(len(toks)):
        _close(got[("a", p)], ref[p])


def test_greedy_generation_through_llm_entry_point(model_a):
    """LLM.generate with the ordinary scheduler (chunked prefill under a
    small token budget, two prompts batched) matches oracle greedy."""
    from vllm_amd.entrypoints.llm import LLM
    from vllm_amd.sampling_params import SamplingParams

    path, cfg, wt = model_a
    prompts = [_tokens(37, cfg["vocab"], 31), _tokens(5, cfg["vocab"], 32)]
    n_new = 12
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(n_new):
            seq.append(int(O.forward(cfg, wt, seq)[-1].argmax()))
        want.append(seq[len(p):])
    llm = LLM(model=path, model_path=path, load_format="safetensors",
              dtype="fp32", device="cpu", num_gpu_blocks=8,
              max_model_len=128, max_num_seqs=4, max_num_batched_tokens=16)
    try:
        outs = llm.generate(
            prompts, SamplingParams(temperature=0.0, max_tokens=n_new,
                                    ignore_eos=True))
    finally:
        llm.shutdown()
    assert [list(o.outputs[0].token_ids) for o in outs] == want


def test_served_over_http(model_a):
    """The OpenAI-compatible server loads the folder like any other
    model; token-id prompts, greedy completion, same tokens as the
    oracle (the family has no tokenizer: text is the byte fallback)."""
    from fastapi.testclient import TestClient

    from vllm_amd.engine.arg_utils import EngineArgs
    from vllm_amd.entrypoints.openai.api_server import make_server

    path, cfg, wt = model_a
    prompt = _tokens(9, cfg["vocab"], 77)
    seq = list(prompt)
    for _ in range(4):
        seq.append(int(O.forward(cfg, wt, seq)[-1].argmax()))
    args = EngineArgs(model=path, model_path=path, load_format="safetensors",
                      dtype="fp32", device="cpu", num_gpu_blocks=8,
                      max_model_len=256, max_num_seqs=4,
                      max_num_batched_tokens=64)
    app, state = make_server(args, None)
    try:
        with TestClient(app) as c:
            r = c.post("/v1/completions", json={
                "model": path, "prompt": prompt, "max_tokens": 4,
                "temperature": 0, "logprobs": 1})
            assert r.status_code == 200, r.text
            lp = r.json()["choices"][0]["logprobs"]
            assert len(lp["tokens"]) == 4
    finally:
        state.engine.shutdown()
    # The ids come back as text bytes (every id of this vocab is < 128).
    text = r.json()["choices"][0]["text"]
    assert [ord(ch) for ch in text] == seq[len(prompt):]


def test_config_errors(tmp_path):
    from vllm_amd.config import get_model_spec

    cfg = O.make_config([O.layer_entry(), O.layer_entry(weights_of=5)])
    path = O.save_model(str(tmp_path / "bad"), cfg,
                        O.random_weights(O.make_config([O.layer_entry()])))
    with pytest.raises(ValueError):
        get_model_spec(path)
