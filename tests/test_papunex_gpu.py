"""Papunex family on the GPU: every HIP kernel against a plain fp32
computation of the same op, then the engine in fp32 and bf16 against
the oracle (tests/papunex_oracle.py) under mixed schedules."""

from __future__ import annotations

import math
import random

import pytest
import torch

from tests import papunex_oracle as O
from tests.gadilix_harness import chunked, run_schedule, whole
from tests.test_papunex import (_latent_plain, _latent_through_cache,
                                _tokens)

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _close(got, ref, tol):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert got.shape == ref.shape
    if ref.numel() == 0:
        return
    err = (got - ref).abs().max().item()
    assert err <= tol * max(1.0, ref.abs().max().item()), err


def _ref_ops():
    from vllm_amd.ops import _torch_ref
    return _torch_ref


@pytest.mark.parametrize("width", [384, 24, 4096, 5000, 33])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_kernels(width, dtype):
    from vllm_amd import ops

    torch.manual_seed(width)
    R = _ref_ops()
    y = (torch.randn(7, width) * 3).to(dtype)
    w = torch.rand(width) + 0.5
    x = torch.randn(7, width)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    _close(ops.rms_norm_cast(x.to(DEV), w.to(DEV), 1e-5, dtype),
           R.rms_norm_cast(x, w, 1e-5, torch.float32), tol)
    xr = x.clone()
    R.add_rms_norm(xr, y, w, 1e-5)
    xg = x.to(DEV)
    copy = ops.add_rms_norm(xg, y.to(DEV), w.to(DEV), 1e-5, dtype)
    _close(xg, xr, 1e-5)
    _close(copy, xr, tol)
    assert copy.dtype == dtype


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels(dtype):
    from vllm_amd import ops

    torch.manual_seed(1)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for n in (1, 7, 1024, 4099):
        x = (torch.randn(3, n) * 2).to(dtype)
        _close(ops.relu2(x.to(DEV)), torch.relu(x.float()) ** 2, tol)
        big = (x * 9).to(dtype)
        _close(ops.logit_softcap(big.to(DEV), 13.0),
               13.0 * torch.tanh(big.float() / 13.0), 1e-5)
    table = torch.randn(50, 36).to(dtype)
    ids = torch.tensor([4, 49, 0, 4, 17])
    _close(ops.scaled_embedding(ids.to(DEV), table.to(DEV), 3.25),
           table[ids].float() * 3.25, 1e-6)
    h = torch.randn(3, 6, 10).to(dtype)          # [H, T, D]
    g = torch.randn(6, 30).to(dtype)
    big = torch.randn(6, 70).to(dtype)
    big[:, 20:50] = g
    got = ops.sigmoid_gate_mul(h.to(DEV).transpose(0, 1),
                               big.to(DEV)[:, 20:50])
    ref = h.float().transpose(0, 1).reshape(6, 30) * torch.sigmoid(g.float())
    _close(got, ref, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_and_cache_write_kernel(dtype):
    from vllm_amd import ops
    from vllm_amd.layers.rotary import PairwiseRotary

    torch.manual_seed(2)
    R_ = _ref_ops()
    T, H, D, R, L, dims = 9, 5, 8, 16, 24, 12
    rot = PairwiseRotary(dims, 10000.0)
    wide = torch.randn(T, H * (D + R) + L + R + 8).to(dtype)
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 1000, 4095, 70000])
    slots = torch.tensor([3, 9, -1, 0, 1, 2, 30, 17, 8])
    w = torch.rand(L) + 0.5
    cache_ref = torch.zeros(2, 16, L + R, dtype=dtype)
    q_ref = wide[:, :H * (D + R)].clone().view(T, H, D + R)
    R_.latent_rope_cache_write(q_ref, wide[:, H * (D + R):H * (D + R) + L + R],
                               w, 1e-5, pos, rot.inv_freq, D, L, cache_ref,
                               slots)
    wg = wide.to(DEV)
    cache = torch.zeros(2, 16, L + R, dtype=dtype, device=DEV)
    qg = wg[:, :H * (D + R)].view(T, H, D + R)
    ops.latent_rope_cache_write(
        qg, wg[:, H * (D + R):H * (D + R) + L + R], w.to(DEV), 1e-5,
        pos.to(DEV), rot.inv_freq.to(DEV), D, L, cache, slots.to(DEV))
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    _close(qg, q_ref, tol)
    _close(cache, cache_ref, tol)
    # A layer that reads another layer's keys only rotates its queries.
    q2 = wide[:, :H * (D + R)].to(DEV).view(T, H, D + R).clone()
    ops.latent_rope_cache_write(q2, None, None, 1e-5, pos.to(DEV),
                                rot.inv_freq.to(DEV), D, L, None, None)
    _close(q2, q_ref, tol)


@pytest.mark.parametrize("L,R,H", [(6, 4, 3), (300, 2, 2), (64, 32, 5),
                                   (5, 0, 1)])
def test_latent_attention_rows_fp32(L, R, H):
    torch.manual_seed(L + R)
    T = 150
    q_abs = torch.randn(T, H, L) * (3.0 / math.sqrt(L))
    q_rot = torch.randn(T, H, R)
    rows = torch.randn(T, L + R)
    sink = torch.randn(H)
    ref = _latent_plain(q_abs, q_rot, rows, 0.5, sink)
    for cuts in ([T], [2, 61, 1, 1, 3, 64, 2, 100], [100] + [1] * 50):
        got = _latent_through_cache(q_abs, q_rot, rows, 0.5, sink, cuts,
                                    bs=64, device=DEV)
        _close(got, ref, 2e-5)


@pytest.mark.parametrize("L,R,H", [(64, 32, 4), (64, 32, 3), (128, 32, 16),
                                   (128, 64, 40), (256, 64, 32),
                                   (512, 64, 128), (512, 64, 1),
                                   (96, 16, 6), (40, 8, 2), (200, 24, 12),
                                   (8, 0, 2), (320, 40, 20), (64, 64, 7)])
def test_latent_attention_tiles_bf16(L, R, H):
    """MFMA tile kernel: prompt portions and decode rows, several
    tokens per workgroup (H < 32), several workgroups per token
    (H > 32), rows narrower than the tile they run on, with a sink."""
    torch.manual_seed(L + R + H)
    T = 140 if H > 8 else 1200     # few heads: also a long context
    q_abs = (torch.randn(T, H, L) * (3.0 / math.sqrt(L))).bfloat16().float()
    q_rot = torch.randn(T, H, R).bfloat16().float()
    rows = torch.randn(T, L + R).bfloat16().float()
    sink = torch.randn(H)
    ref = _latent_plain(q_abs, q_rot, rows, 0.5, sink)
    for cuts in ([T], [2, 61, 1, 1, 3, 64, 2, 100, 900, 2000],
                 [T - 50] + [1] * 50):
        got = _latent_through_cache(q_abs, q_rot, rows, 0.5, sink, cuts,
                                    bs=64, device=DEV,
                                    dtype=torch.bfloat16)
        _close(got, ref, 2e-2)


def test_latent_attention_batch_of_decodes_and_portions():
    """Decode rows of unequal context (one to five key partitions)
    beside two prompt portions, shuffled pages."""
    from vllm_amd import ops

    torch.manual_seed(4)
    H, L, R, bs = 4, 64, 32, 64
    ctxs = [1100, 3, 64, 700, 130]       # contexts after this step
    news = [1, 1, 1, 37, 130]            # tokens of this step
    nb = sum(-(-c // bs) for c in ctxs) + 2
    for dtype, tol in ((torch.bfloat16, 2e-2), (torch.float32, 2e-5)):
        cache = torch.zeros(nb, bs, L + R, dtype=dtype, device=DEV)
        pages = list(range(nb))
        random.Random(1).shuffle(pages)
        bt = torch.zeros(len(ctxs), max(-(-c // bs) for c in ctxs),
                         dtype=torch.int32)
        qa, qr, refs, qsl = [], [], [], [0]
        for i, (c, n) in enumerate(zip(ctxs, news)):
            rows = torch.randn(c, L + R).to(dtype).float()
            mine = [pages.pop() for _ in range(-(-c // bs))]
            bt[i, :len(mine)] = torch.tensor(mine)
            pos = torch.arange(c)
            slot = torch.tensor(mine)[pos // bs] * bs + pos % bs
            cache.view(-1, L + R)[slot.to(DEV)] = rows.to(DEV, dtype)
            a = (torch.randn(c, H, L) * 0.4).to(dtype).float()
            r = torch.randn(c, H, R).to(dtype).float()
            sink = torch.linspace(-1, 1, H)
            refs.append(_latent_plain(a, r, rows, 0.3, sink)[c - n:])
            qa.append(a[c - n:])
            qr.append(r[c - n:])
            qsl.append(qsl[-1] + n)
        got = ops.latent_attention(
            torch.cat(qa).to(DEV, dtype), torch.cat(qr).to(DEV, dtype),
            cache, bt.to(DEV),
            torch.tensor(qsl, dtype=torch.int32, device=DEV),
            torch.tensor(ctxs, dtype=torch.int32, device=DEV), 0.3,
            sink=sink.to(DEV), num_decodes=3, max_seq_len=max(ctxs),
            max_query_len=max(news))
        _close(got, torch.cat(refs), tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [1, 2, 4])
def test_conv_kernel(K, dtype):
    from vllm_amd import ops

    torch.manual_seed(K)
    R = _ref_ops()
    C = 300
    lens = [1, 5, 1, 40, 2]
    x = torch.randn(sum(lens), C + 16).to(dtype)
    w = torch.randn(C, K).to(dtype)
    b = torch.randn(C).to(dtype)
    qsl = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)),
                       dtype=torch.int32)
    rows = torch.tensor([4, 0, 2, 5, 1])
    st_ref = torch.randn(6, C, K - 1).to(dtype)
    st = st_ref.clone().to(DEV)
    ref = R.causal_conv_silu(x[:, 8:8 + C], w, b, st_ref, rows, qsl,
                             torch.float32)
    got = ops.causal_conv_silu(x.to(DEV)[:, 8:8 + C], w.to(DEV), b.to(DEV),
                               st, rows.to(DEV), qsl.to(DEV),
                               out_dtype=torch.float32)
    _close(got, ref, 1e-5 if dtype == torch.float32 else 1e-2)
    _close(st, st_ref, 0)
    got = ops.causal_conv_silu(x.to(DEV)[:, 8:8 + C], w.to(DEV), b.to(DEV),
                               None, None, qsl.to(DEV))
    assert got.dtype == dtype


@pytest.mark.parametrize("lens", [[1, 1, 70, 33, 2], [1, 700, 256, 2, 257]])
@pytest.mark.parametrize("Hm,P,G,N", [(8, 32, 4, 40), (4, 64, 1, 128),
                                      (3, 5, 3, 3), (2, 100, 1, 200),
                                      (6, 16, 2, 17)])
def test_scan_kernel(Hm, P, G, N, lens):
    """Short portions run sequentially; a portion longer than 256 tokens
    switches the whole batch to parallel segments with a carry pass."""
    from vllm_amd import ops

    torch.manual_seed(Hm * P)
    R = _ref_ops()
    T = sum(lens)
    xbc = torch.randn(T, Hm * P + 2 * G * N)
    dt = torch.randn(T, Hm + 4)
    dt_bias, a_log = torch.randn(Hm) - 1, torch.randn(Hm) * 0.5
    d_skip = torch.randn(Hm)
    qsl = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)),
                       dtype=torch.int32)
    rows = torch.tensor([3, 1, 0, 5, 2])
    st_ref = torch.randn(6, Hm, P, N)
    st = st_ref.clone().to(DEV)
    ref = R.ssd_scan(xbc, Hm, P, G, N, dt[:, 2:2 + Hm], dt_bias, a_log,
                     d_skip, st_ref, rows, qsl)
    got = ops.ssd_scan(xbc.to(DEV), Hm, P, G, N,
                       dt.to(DEV)[:, 2:2 + Hm], dt_bias.to(DEV),
                       a_log.to(DEV), d_skip.to(DEV), st, rows.to(DEV),
                       qsl.to(DEV), max_query_len=max(lens))
    _close(got, ref, 5e-5)
    _close(st, st_ref, 5e-5)
    got = ops.ssd_scan(xbc.to(DEV), Hm, P, G, N,
                       dt.to(DEV)[:, 2:2 + Hm].bfloat16(), dt_bias.to(DEV),
                       a_log.to(DEV), d_skip.to(DEV), None, None,
                       qsl.to(DEV))
    assert got.shape == (T, Hm, P)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_group_norm_kernel(dtype):
    from vllm_amd import ops

    R = _ref_ops()
    torch.manual_seed(3)
    for W, groups in ((256, 2), (12, 3), (1200, 1)):
        y = torch.randn(5, W)
        z = torch.randn(5, W + 8).to(dtype)
        w = torch.rand(W) + 0.5
        ref = R.gated_group_rms_norm(y, z[:, 8:], w, 1e-5, groups,
                                     torch.float32)
        got = ops.gated_group_rms_norm(y.to(DEV), z.to(DEV)[:, 8:],
                                       w.to(DEV), 1e-5, groups, dtype)
        _close(got, ref, 1e-5 if dtype == torch.float32 else 1e-2)


def test_squared_relu_experts_on_gpu():
    from vllm_amd import ops

    torch.manual_seed(0)
    R = _ref_ops()
    for dtype, tol in ((torch.float32, 1e-4), (torch.bfloat16, 3e-2)):
        for E, ff, width, T in ((4, 24, 40, 9), (8, 128, 256, 70)):
            up = (torch.randn(E, ff, width) / math.sqrt(width)).to(dtype)
            down = (torch.randn(E, width, ff) / math.sqrt(ff)).to(dtype)
            x = torch.randn(T, width).to(dtype)
            w = torch.rand(T, 2)
            ids = torch.stack([torch.randperm(E)[:2]
                               for _ in range(T)]).int()
            ref = R.fused_moe(x.float(), up.float(), down.float(), w, ids,
                              "relu2")
            got = ops.fused_moe(x.to(DEV), up.to(DEV), down.to(DEV),
                                w.to(DEV), ids.to(DEV), activation="relu2")
            _close(got, ref, tol)


# ---------------------------------------------------------------------
# Engine on the GPU.

@pytest.fixture(scope="module")
def model_g(tmp_path_factory):
    """Shapes of the MFMA tile kernel (kv_rank 64, rot_dim 32) next to
    off-template ones, both mixers, all feed-forward kinds."""
    layers = [
        O.latent_entry(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64,
                       rot_dims=32, base=10000.0, mlp="dense", ff=64),
        O.mamba_entry(heads=4, vdim=16, state=24, groups=2, conv=4,
                      norm_groups=2, mlp="moe", ff=32, experts=6, top=2,
                      router_scale=1.3, shared_ff=32),
        O.latent_entry(heads=6, dim=8, rot_dim=32, vdim=8, kv_rank=64,
                       rot_dims=32, base=10000.0, kv_from=0, mlp=None),
        O.latent_entry(heads=3, dim=8, rot_dim=6, vdim=10, kv_rank=12,
                       rot_dims=4, mlp="moe", ff=16, experts=3, top=3,
                       shared_ff=0),
        O.mamba_entry(heads=2, vdim=40, state=20, groups=1, conv=2,
                      norm_groups=1, mlp="dense", ff=32),
    ]
    cfg = O.make_config(layers, vocab=64, width=64, embed_scale=4.0,
                        softcap=25.0)
    wt = O.random_weights(cfg, seed=7)
    path = O.save_model(str(tmp_path_factory.mktemp("papunex_g")), cfg, wt)
    return path, cfg, wt


def _mixed_steps(reqs):
    at = {k: 0 for k in reqs}
    plan = [{"a": 30, "b": 1, "c": 2}, {"a": 1, "c": 64, "d": 1},
            {"a": 1, "b": 3, "c": 1}, {"b": 5, "c": 63}, {"a": 1, "c": 1},
            {"a": 1, "c": 1}, {"a": 0}, {"c": 0}]
    steps = []
    for st in plan:
        ent, end = [], []
        for k, n in st.items():
            if at[k] >= len(reqs[k]):
                continue
            n = min(n, len(reqs[k]) - at[k]) if n else len(reqs[k]) - at[k]
            ent.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        steps.append((ent, end))
    assert all(at[k] == len(reqs[k]) for k in reqs)
    return steps


def _compare_positions(got, refs, dtype):
    """fp32: every position within 3e-4 of the largest logit. bf16:
    rounding can flip a close routing decision of this random model,
    which moves one position's logits by a discrete step, so the
    centred RMS error is held to what the torch reference ops show in
    bf16 on the same model (median 0.019, 95th percentile 0.07, worst
    0.35), with some room."""
    errs = []
    for k, ref in refs.items():
        for p in range(ref.shape[0]):
            d = got[(k, p)] - ref[p]
            if dtype == "float32":
                err = d.abs().max().item()
                assert err <= 3e-4 * max(1.0, ref[p].abs().max().item()), \
                    (k, p, err)
            else:
                d = d - d.mean()
                scale = (ref[p] - ref[p].mean()).pow(2).mean().sqrt().item()
                errs.append(d.pow(2).mean().sqrt().item() / max(scale, 1e-3))
    if errs:
        errs.sort()
        assert errs[len(errs) // 2] <= 0.03, errs[len(errs) // 2]
        assert errs[int(0.95 * len(errs))] <= 0.12, errs[-10:]
        assert errs[-1] <= 0.6, errs[-10:]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_on_gpu(model_g, dtype):
    path, cfg, wt = model_g
    vocab = cfg["vocab"]
    reqs = {"a": _tokens(70, vocab, 1), "b": _tokens(9, vocab, 2),
            "c": _tokens(150, vocab, 3), "d": _tokens(1, vocab, 4)}
    refs = {k: O.forward(cfg, wt, v) for k, v in reqs.items()}
    got, _ = run_schedule(path, _mixed_steps(reqs), dtype=dtype,
                          max_tokens=448, device=DEV)
    _compare_positions(got, refs, dtype)
    # Rows and pages reused by later requests.
    steps = []
    later = {}
    for i in range(6):
        toks = _tokens(40 + 9 * i, vocab, 50 + i)
        later[f"r{i}"] = toks
        steps += chunked(f"r{i}", toks, [17, 1, 1])
    got, _ = run_schedule(path, steps, dtype=dtype, max_tokens=128,
                          device=DEV)
    _compare_positions(
        got, {k: O.forward(cfg, wt, t) for k, t in later.items()}, dtype)


def test_engine_rows_narrower_than_the_tile(tmp_path):
    """Latent rows that run on a wider tile of the MFMA kernel (96 + 16
    on 128 + 32, 40 + 8 on 64 + 32) with head sizes that leave the
    rotated query part off a 16 B boundary, through the engine in bf16
    and fp32, one request in portions beside decode rows."""
    layers = [
        O.latent_entry(heads=5, dim=20, rot_dim=16, vdim=12, kv_rank=96,
                       rot_dims=12, base=5000.0, mlp="dense", ff=48),
        O.latent_entry(heads=3, dim=24, rot_dim=16, vdim=20, kv_rank=96,
                       rot_dims=12, base=5000.0, kv_from=0, mlp="moe",
                       ff=24, experts=4, top=2, shared_ff=16),
        O.latent_entry(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=40,
                       mlp=None),
    ]
    cfg = O.make_config(layers, vocab=50, width=40, embed_scale=2.0,
                        softcap=18.0)
    wt = O.random_weights(cfg, seed=11)
    path = O.save_model(str(tmp_path / "m"), cfg, wt)
    reqs = {"a": _tokens(70, 50, 1), "b": _tokens(9, 50, 2),
            "c": _tokens(150, 50, 3), "d": _tokens(1, 50, 4)}
    refs = {k: O.forward(cfg, wt, v) for k, v in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        got, _ = run_schedule(path, _mixed_steps(reqs), dtype=dtype,
                              max_tokens=448, device=DEV)
        _compare_positions(got, refs, dtype)


def test_greedy_generation_on_gpu(model_g):
    from vllm_amd.entrypoints.llm import LLM
    from vllm_amd.sampling_params import SamplingParams

    path, cfg, wt = model_g
    prompts = [_tokens(12, cfg["vocab"], 40), _tokens(3, cfg["vocab"], 41)]
    llm = LLM(model=path, model_path=path, load_format="safetensors",
              dtype="fp32", num_gpu_blocks=8, max_model_len=128,
              max_num_seqs=4, max_num_batched_tokens=8)
    try:
        outs = llm.generate(
            prompts, SamplingParams(temperature=0.0, max_tokens=6,
                                    ignore_eos=True))
    finally:
        llm.shutdown()
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.outputs[0].token_ids:
            logits = O.forward(cfg, wt, seq)[-1]
            top2 = logits.topk(2).values
            if float(top2[0] - top2[1]) > 1e-3:
                assert tok == int(logits.argmax())
            seq.append(tok)


def test_captured_decode_matches_eager(tmp_path):
    """One-token steps replayed from captured hipGraphs (batch buckets
    with padded rows, requests joining and leaving, state rows staged
    per step, a context of several key partitions) against the eager
    engine: both run the same kernels, so they agree to rounding of
    the library GEMMs' algorithm choice."""
    layers = [
        O.latent_entry(heads=4, dim=16, rot_dim=32, vdim=32, kv_rank=64,
                       rot_dims=32, base=10000.0, mlp="moe", ff=128,
                       experts=6, top=2, shared_ff=128),
        O.mamba_entry(heads=4, vdim=32, state=24, groups=2, conv=4,
                      norm_groups=2, mlp="dense", ff=128),
        O.latent_entry(heads=8, dim=8, rot_dim=32, vdim=16, kv_rank=64,
                       rot_dims=32, base=10000.0, kv_from=0, mlp=None),
        O.latent_entry(heads=2, dim=8, rot_dim=6, vdim=12, kv_rank=20,
                       rot_dims=6, mlp="moe", ff=128, experts=4, top=1,
                       shared_ff=0),
    ]
    cfg = O.make_config(layers, vocab=80, width=128, embed_scale=3.0,
                        softcap=25.0)
    wt = O.random_weights(cfg, seed=5)
    path = O.save_model(str(tmp_path / "m"), cfg, wt)
    reqs = {"a": _tokens(1080, 80, 41), "b": _tokens(90, 80, 42),
            "c": _tokens(70, 80, 43)}
    steps = [([("a", reqs["a"][:1000], [999]),
               ("b", reqs["b"][:50], [49])], [])]
    for i in range(40):                       # two decode rows
        steps.append(([("a", reqs["a"][1000 + i:1001 + i], [0]),
                       ("b", reqs["b"][50 + i:51 + i], [0])],
                      ["b"] if i == 39 else []))
    steps.append(([("c", reqs["c"][:60], [59])], []))
    for i in range(10):                       # other rows, other bucket
        steps.append(([("a", reqs["a"][1040 + i:1041 + i], [0]),
                       ("c", reqs["c"][60 + i:61 + i], [0])],
                      ["a", "c"] if i == 9 else []))
    for i in range(30):                       # one row alone
        steps.append(([("d", _tokens(1, 80, 100 + i), [0])],
                      ["d"] if i == 29 else []))
    graph, core = run_schedule(path, steps, dtype="bfloat16",
                               max_tokens=1408, device=DEV,
                               enforce_eager=False)
    assert core.worker.runner.graph_runner is not None
    assert core.worker.runner.graph_runner.graphs, "nothing was captured"
    eager, _ = run_schedule(path, steps, dtype="bfloat16", max_tokens=1408,
                            device=DEV)
    assert graph.keys() == eager.keys()
    errs = []
    for key, got in graph.items():
        d = got - eager[key]
        d = d - d.mean()
        scale = (eager[key] - eager[key].mean()).pow(2).mean().sqrt().item()
        errs.append(d.pow(2).mean().sqrt().item() / max(scale, 1e-3))
    errs.sort()
    assert errs[len(errs) // 2] <= 0.02, errs[len(errs) // 2]
    assert errs[int(0.95 * len(errs))] <= 0.1, errs[-10:]
