"""Prefill and decode throughput of a model family beside the closest
existing family at equal active size (random weights, one GPU).

    python bench.py --compare-family gadilix [--compare-sizes small,medium]
    python bench.py --compare-family papunex [--compare-sizes small,medium]

"papunex" builds three engines per size: an all-latent-attention
Papunex stack, a hybrid one (latent attention and Mamba-2 layers
alternating) and a DeepSeek-structured stack (latent attention of the
same kv_rank / rotated width / head sizes, routed SwiGLU experts plus a
shared one) whose expert width is 2/3 of the squared-relu experts', so
both move the same number of expert parameters per token.

For every "gadilix" size it builds two engines in turn — the Gadilix stack
(sliding window + pooled far blocks, token-table MoE + shared expert)
and a Mixtral-structured stack (GQA attention with the same sliding
window, learned-router MoE) whose per-token active expert width matches
— and measures

  prefill: tokens/s of `prefill_batch` prompts of `prompt_len` tokens
           scheduled as one chunked-prefill stream,
  decode:  tokens/s of `decode_steps` full-batch decode steps at
           context ~= prompt_len.

One JSON line per (family, size, phase) goes to stdout. The default
bench.py workload and its one-line output are untouched.
"""

from __future__ import annotations

import json
import os
import tempfile
import time

import numpy as np
import torch

SIZES = {
    # width, layers, heads, kv_heads, head_dim, experts, top, ff (per
    # routed expert), window, pool, vocab
    "small": dict(width=2048, layers=4, heads=16, kv_heads=4, dim=128,
                  experts=8, top=2, ff=1024, window=1024, pool=64,
                  vocab=32000),
    "medium": dict(width=4096, layers=2, heads=32, kv_heads=8, dim=128,
                   experts=8, top=2, ff=2048, window=2048, pool=64,
                   vocab=32000),
}


PAPUNEX_SIZES = {
    # Latent attention with the usual 512 + 64 cache row; Mamba-2 layers
    # of inner width 2 * width, 64-wide heads, state 128.
    "small": dict(width=2048, layers=4, heads=16, dim=128, rot_dim=64,
                  vdim=128, kv_rank=512, experts=8, top=2, ff=1536,
                  shared_ff=1536, ssm_state=128, ssm_groups=8,
                  vocab=32000),
    "medium": dict(width=4096, layers=2, heads=32, dim=128, rot_dim=64,
                   vdim=128, kv_rank=512, experts=8, top=2, ff=3072,
                   shared_ff=3072, ssm_state=128, ssm_groups=8,
                   vocab=32000),
}


def _papunex_dir(s: dict, hybrid: bool) -> str:
    mlp = {"kind": "moe", "expert": {"ff": s["ff"]},
           "router": {"experts": s["experts"], "top": s["top"],
                      "scale": 1.0},
           "shared": {"ff": s["shared_ff"]}}
    att = {"type": "latent_attention",
           "mixer": {"heads": s["heads"], "dim": s["dim"],
                     "rot_dim": s["rot_dim"], "vdim": s["vdim"],
                     "kv_rank": s["kv_rank"],
                     "rot": {"base": 10000.0, "dims": s["rot_dim"]},
                     "scale": (s["dim"] + s["rot_dim"]) ** -0.5},
           "mlp": mlp}
    ssm = {"type": "mamba2",
           "mixer": {"heads": 2 * s["width"] // 64, "vdim": 64,
                     "state": s["ssm_state"], "groups": s["ssm_groups"],
                     "conv": 4, "norm_groups": s["ssm_groups"]},
           "mlp": mlp}
    layers = [ssm if hybrid and i % 2 else att
              for i in range(s["layers"])]
    cfg = {"architecture": "Papunex", "vocab": s["vocab"],
           "width": s["width"], "embedding": {"scale": 1.0},
           "norm": {"eps": 1e-5}, "logit_softcap": 30.0, "layers": layers}
    d = tempfile.mkdtemp(prefix="papunex_bench_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    return d


def _deepseek_spec(s: dict):
    from vllm_amd.config import ModelSpec

    inter = s["ff"] * 2 // 3
    return ModelSpec(
        name="deepseek-like", architecture="deepseek",
        vocab_size=s["vocab"], hidden_size=s["width"],
        intermediate_size=inter, num_layers=s["layers"],
        num_heads=s["heads"], num_kv_heads=s["heads"],
        head_dim=s["dim"] + s["rot_dim"], rope_theta=10000.0,
        max_position_embeddings=1 << 17, num_experts=s["experts"],
        num_experts_per_tok=s["top"], moe_intermediate_size=inter,
        num_shared_experts=1, first_dense_layers=0,
        scoring_func="softmax", q_lora_rank=0, kv_lora_rank=s["kv_rank"],
        qk_nope_head_dim=s["dim"], qk_rope_head_dim=s["rot_dim"],
        v_head_dim=s["vdim"])


def _gadilix_dir(s: dict) -> str:
    layer = {
        "type": "attention",
        "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"],
                  "dim": s["dim"], "vdim": s["dim"],
                  "scale": s["dim"] ** -0.5,
                  "mask": {"size": s["window"], "pool": s["pool"]}},
        "mlp": {"kind": "moe", "expert": {"ff": s["ff"]},
                "router": {"experts": s["experts"], "top": s["top"]},
                "shared": {"ff": s["ff"]}},
    }
    cfg = {"architecture": "Gadilix", "vocab": s["vocab"],
           "width": s["width"], "residual_mult": 0.5,
           "norm": {"eps": 1e-5}, "layers": [layer] * s["layers"]}
    d = tempfile.mkdtemp(prefix="gadilix_bench_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    return d


def _mixtral_spec(s: dict):
    from vllm_amd.config import ModelSpec

    # Active expert width per token equal to the other stack's
    # top * ff + shared ff.
    inter = s["ff"] + s["ff"] // s["top"]
    return ModelSpec(
        name="mixtral-like", architecture="mixtral", vocab_size=s["vocab"],
        hidden_size=s["width"], intermediate_size=inter,
        num_layers=s["layers"], num_heads=s["heads"],
        num_kv_heads=s["kv_heads"], head_dim=s["dim"],
        max_position_embeddings=1 << 20, num_experts=s["experts"],
        num_experts_per_tok=s["top"], moe_intermediate_size=inter,
        sliding_window=s["window"])


def _engine(family: str, s: dict, max_len: int, batch: int, tokens: int):
    from vllm_amd.config import (CacheConfig, DeviceConfig, EngineConfig,
                                 ModelConfig, ParallelConfig,
                                 SchedulerConfig)
    from vllm_amd.engine.core import EngineCore

    if family == "gadilix":
        mc = ModelConfig(model=_gadilix_dir(s), dtype="bf16",
                         max_model_len=max_len, load_format="dummy")
    elif family in ("papunex", "papunex-hybrid"):
        mc = ModelConfig(model=_papunex_dir(s, family.endswith("hybrid")),
                         dtype="bf16", max_model_len=max_len,
                         load_format="dummy")
    elif family == "deepseek-like":
        mc = ModelConfig(model="deepseek-like", dtype="bf16",
                         max_model_len=max_len, load_format="dummy",
                         spec=_deepseek_spec(s))
    else:
        mc = ModelConfig(model="mixtral-like", dtype="bf16",
                         max_model_len=max_len, load_format="dummy",
                         spec=_mixtral_spec(s))
    blocks = batch * (-(-max_len // 64) + 1)
    return EngineCore(EngineConfig(
        model_config=mc,
        cache_config=CacheConfig(block_size=64, num_gpu_blocks=blocks,
                                 enable_prefix_caching=False),
        scheduler_config=SchedulerConfig(
            max_num_batched_tokens=tokens, max_num_seqs=batch,
            enable_chunked_prefill=True, async_scheduling=False),
        parallel_config=ParallelConfig(),
        device_config=DeviceConfig(device="cuda"),
    ))


def _run(family: str, name: str, s: dict, prompt_len: int,
         prefill_batch: int, decode_batch: int, decode_steps: int,
         chunk_tokens: int):
    from vllm_amd.request import Request
    from vllm_amd.sampling_params import SamplingParams

    batch = max(prefill_batch, decode_batch)
    max_len = prompt_len + decode_steps + 80
    eng = _engine(family, s, max_len, batch, chunk_tokens)
    rng = np.random.default_rng(0)
    params = SamplingParams(temperature=0.0, max_tokens=decode_steps + 64,
                            ignore_eos=True, detokenize=False)

    def add(n, tag):
        for i in range(n):
            eng.add_request(Request(
                f"{tag}{i}", rng.integers(16, s["vocab"] - 16,
                                          size=prompt_len).tolist(),
                params, arrival_time=time.time()))

    def drain_prefill(seen, n_reqs):
        """Step until n_reqs requests have produced their first token."""
        while len(seen) < n_reqs:
            for out in eng.step():
                if out.new_token_ids:
                    seen.add(out.req_id)

    def one_pass(tag):
        """The whole workload once: timed prefill of `prefill_batch`
        prompts, the rest of the decode batch admitted, then timed
        full-batch decode steps; every request dropped at the end."""
        seen: set = set()
        add(prefill_batch, tag + "p")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        drain_prefill(seen, prefill_batch)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        res = [("prefill", prefill_batch * prompt_len / dt, dt)]
        if decode_batch > prefill_batch:
            add(decode_batch - prefill_batch, tag + "d")
            drain_prefill(seen, decode_batch)
        for _ in range(4):
            eng.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        toks = 0
        for _ in range(decode_steps):
            for out in eng.step():
                toks += len(out.new_token_ids)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        res.append(("decode", toks / dt, dt))
        eng.abort_requests(
            [f"{tag}p{i}" for i in range(prefill_batch)]
            + [f"{tag}d{i}" for i in range(decode_batch - prefill_batch)])
        eng.step()
        return res

    # The first pass is untimed: the scheduler cuts both passes into
    # the same steps, so every GEMM shape of the timed pass has had its
    # algorithm chosen and the allocator holds its buffers.
    one_pass("w")
    results = one_pass("t")
    eng.shutdown()
    for phase, tps, secs in results:
        print(json.dumps({
            "family": family, "size": name, "phase": phase,
            "tokens_per_s": round(tps, 1), "seconds": round(secs, 4),
            "config": {**s, "prompt_len": prompt_len,
                       "prefill_batch": prefill_batch,
                       "decode_batch": decode_batch,
                       "decode_steps": decode_steps,
                       "chunk_tokens": chunk_tokens},
            "dtype": "bf16", "data": "synthetic, random-init weights",
        }), flush=True)
    del eng
    torch.cuda.empty_cache()


def main(family: str, sizes: str, prompt_len: int = 4096,
         prefill_batch: int = 4, decode_batch: int = 64,
         decode_steps: int = 32, chunk_tokens: int = 8192) -> None:
    if family not in ("gadilix", "papunex"):
        raise SystemExit(
            f"unknown family {family!r} (known: gadilix, papunex)")
    if not torch.cuda.is_available():
        raise SystemExit("--compare-family needs a GPU")
    table, fams = ((SIZES, ("gadilix", "mixtral-like"))
                   if family == "gadilix" else
                   (PAPUNEX_SIZES,
                    ("papunex", "papunex-hybrid", "deepseek-like")))
    only = os.environ.get("VLLM_AMD_COMPARE_ONLY")
    if only:
        fams = tuple(f for f in fams if f in only.split(","))
    for name in sizes.split(","):
        s = table[name]
        for fam in fams:
            _run(fam, name, s, prompt_len, prefill_batch, decode_batch,
                 decode_steps, chunk_tokens)
