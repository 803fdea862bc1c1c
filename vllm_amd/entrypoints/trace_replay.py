"""Replay a token trace through the engine and dump raw logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR \\
                  --max-tokens N

Standard input carries one JSON object per step,

    {"step": 3, "entries": [{"id": "a", "tokens": [5, 17], "want": [1]}],
     "end": ["b"]}

'entries' brings each request's next tokens (a request is admitted at
its first entry and may sit out any step); 'want' lists offsets into
those tokens whose logits are asked for; 'end' names requests to drop
after the step. Nothing is sampled. For a step that wants logits the
rows are written to OUT/<step>.f32 (little-endian fp32 [wanted, vocab],
in entry order); after every step 'done <step>' goes to standard output.

The replay is a client of the ordinary engine: requests are admitted
with an open (streamed) prompt, each step appends the new tokens and
logit taps through the scheduler, EngineCore.step() schedules, runs
the model runner and returns the tapped logits, and ended requests are
aborted so their pages and state rows go back to the pools. The KV
pool holds exactly --max-tokens tokens (rounded up to pages) and four
request rows.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

MAX_LIVE_REQUESTS = 4


def build_core(model_dir: str, dtype: str, max_tokens: int,
               device: str = "auto", enforce_eager: bool = True):
    from vllm_amd.engine.arg_utils import EngineArgs
    from vllm_amd.engine.core import EngineCore

    block_size = 64
    num_blocks = max(1, -(-max_tokens // block_size))
    args = EngineArgs(
        model=model_dir,
        model_path=model_dir,
        load_format="safetensors",
        dtype={"bfloat16": "bf16", "float32": "fp32"}[dtype],
        block_size=block_size,
        num_gpu_blocks=num_blocks,
        max_model_len=num_blocks * block_size,
        max_num_seqs=MAX_LIVE_REQUESTS,
        max_num_batched_tokens=num_blocks * block_size,
        enable_prefix_caching=False,
        async_scheduling=False,
        # Eager by default: a replay is short and its batch shapes
        # change every step, so captures would not pay for themselves.
        enforce_eager=enforce_eager,
        device=device,
    )
    return EngineCore(args.create_engine_config())


def replay(core, lines, out_dir: str, emit) -> None:
    from vllm_amd.request import Request
    from vllm_amd.sampling_params import SamplingParams

    sched = core.scheduler
    seen_len: dict[str, int] = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        order: list[tuple[str, int]] = []
        for ent in step.get("entries", []):
            rid, toks = ent["id"], list(ent["tokens"])
            want = list(ent.get("want", []))
            if not toks:
                continue
            base = seen_len.get(rid)
            if base is None:
                core.add_request(Request(
                    rid, toks,
                    SamplingParams(temperature=0.0, max_tokens=1),
                    prompt_open=True, logit_taps=want))
                seen_len[rid] = len(toks)
            else:
                sched.extend_prompt(rid, toks,
                                    logit_taps=[base + w for w in want])
                seen_len[rid] = base + len(toks)
            if want:
                order.append((rid, len(want)))
        got: dict = {}
        if step.get("entries"):
            for out in core.step():
                if out.tapped_logits is not None:
                    got[out.req_id] = out.tapped_logits
        if order:
            rows = []
            for rid, n in order:
                t = got.get(rid)
                if t is None or t.shape[0] != n:
                    raise RuntimeError(
                        f"step {step['step']}: request {rid} was not run "
                        "whole in this step (pool too small?)")
                rows.append(t.numpy())
            data = np.ascontiguousarray(
                np.concatenate(rows, axis=0), dtype="<f4")
            path = os.path.join(out_dir, f"{step['step']}.f32")
            with open(path + ".part", "wb") as f:
                f.write(data.tobytes())
            os.replace(path + ".part", path)
        ended = [r for r in step.get("end", []) if r in seen_len]
        if ended:
            core.abort_requests(ended)
            for r in ended:
                sched.release_request(r)
                del seen_len[r]
        emit(f"done {step['step']}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(
        prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True,
                    help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"],
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens the KV pool holds (rounded up to pages)")
    ap.add_argument("--device", default="auto",
                    choices=["auto", "cuda", "cpu"])
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    core = build_core(a.model, a.dtype, a.max_tokens, a.device)

    def emit(text: str) -> None:
        sys.stdout.write(text + "\n")
        sys.stdout.flush()

    try:
        replay(core, sys.stdin, a.out, emit)
    finally:
        core.shutdown()
    return 0


if __name__ == "__main__":
    sys.exit(main())
