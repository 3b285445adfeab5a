"""Replay a recorded schedule through the engine, token ids in, logits out.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N  < steps.jsonl

Every input line is one engine step, ``{"step": n, "entries": [{"id", "tokens", "want"}, ...], "end": [ids]}``:
each entry gives a request its next tokens (a request is admitted at its first entry and may sit steps out), ``want``
lists the places among those tokens whose logits are written, as little-endian fp32 ``[wanted, vocab]`` in the order
of the entries, to ``<out>/<step>.f32``; ``end`` names the requests whose blocks and state slot go back to the pools
after the step.  After each step the line ``done <step>`` is printed.  Nothing is sampled.

The steps go through ``EngineCore.step_forced``: the scheduler's block and row bookkeeping, the workers' persistent
batch, the model runner and its kernels are the ones generation uses; only the choice of how many tokens each request
runs is taken from the input instead of the token budget.  The KV pool is sized for ``--max-tokens`` tokens (rounded
up to whole blocks per request), the batch for ``--max-seqs`` live requests.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, List, Optional

import numpy as np


def add_args(p: argparse.ArgumentParser) -> argparse.ArgumentParser:
    p.add_argument("--model", required=True, help="directory with config.json and model.safetensors")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float16", "float32"])
    p.add_argument("--out", required=True, help="directory the logits files are written to")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time, each request rounded up to a multiple of 64")
    p.add_argument("--max-seqs", type=int, default=4, help="most requests live at any time")
    p.add_argument("--device", default="auto", choices=["auto", "cuda", "cpu"])
    p.add_argument("--block-size", type=int, default=None)
    p.add_argument("--enforce-eager", action="store_true", help="no hipGraph replay of decode steps")
    return p


def ensure_native_libraries(device: str) -> None:
    """A fresh checkout has no built libraries: compile them once, in-tree, before the first GPU step."""
    if device != "cuda":
        return
    from ..ops import hip
    if not os.path.exists(hip._LIB_PATH):
        from ..build import build
        print("building the kernel library (first run in this checkout)", file=sys.stderr, flush=True)
        build(force=False, verbose=False, only=("ops",))


def make_core(args):
    import torch
    from ..engine.arg_utils import EngineArgs
    from ..engine.core import EngineCore
    device = args.device
    if device == "auto":
        device = "cuda" if torch.cuda.device_count() > 0 else "cpu"
    ensure_native_libraries(device)
    block = args.block_size or (64 if device == "cuda" else 16)
    if 64 % block and block % 64:
        raise ValueError("--block-size must divide or be a multiple of 64")
    unit = max(block, 64)
    pool_tokens = -(-int(args.max_tokens) // unit) * unit
    ea = EngineArgs(model=args.model, dtype=args.dtype, device=device, block_size=block,
                    max_num_seqs=int(args.max_seqs), enable_prefix_caching=False,
                    num_gpu_blocks_override=pool_tokens // block, enforce_eager=bool(args.enforce_eager),
                    max_num_batched_tokens=max(pool_tokens, 64), load_format="safetensors")
    cfg = ea.create_engine_config()
    mc = cfg.model_config
    mc.max_model_len = min(int(mc.max_model_len), pool_tokens)
    cfg.scheduler_config.max_model_len = mc.max_model_len
    cfg.observability_config.collect_step_timing = False
    return EngineCore(cfg)


def replay(core, lines, out_dir: str, say=print) -> None:
    from ..engine.request import Request, RequestStatus
    from ..sampling_params import SamplingParams
    os.makedirs(out_dir, exist_ok=True)
    live = set()
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        plan: Dict[str, int] = {}
        wanted: Dict[str, List[int]] = {}
        for e in step.get("entries") or []:
            rid, toks = str(e["id"]), [int(t) for t in e["tokens"]]
            if not toks:
                continue
            if rid in live:
                core.extend_request(rid, toks)
            else:
                core.add_request(Request(rid, toks, SamplingParams(temperature=0.0, max_tokens=None, score_only=True,
                                                                   ignore_eos=True)))
                live.add(rid)
            plan[rid] = len(toks)
            if e.get("want"):
                wanted[rid] = [int(k) for k in e["want"]]
        reply = core.step_forced(plan, wanted)[1] if plan else None
        if wanted:
            got = (reply.logits if reply is not None else None) or {}
            rows = [np.asarray(got[rid], dtype="<f4") for rid in wanted]
            tmp = os.path.join(out_dir, f".{step['step']}.part")
            with open(tmp, "wb") as f:
                f.write(np.ascontiguousarray(np.concatenate(rows, 0)).tobytes())
            os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
        ended = [str(r) for r in step.get("end") or [] if str(r) in live]
        if ended:
            core.finish_requests(ended, RequestStatus.FINISHED_ABORTED)
            live.difference_update(ended)
        say(f"done {step['step']}")


def main(argv: Optional[List[str]] = None) -> int:
    args = add_args(argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])).parse_args(argv)
    os.environ.setdefault("VLLM_LOGGING_LEVEL", "WARNING")
    core = make_core(args)
    try:
        replay(core, sys.stdin, args.out, say=lambda s: print(s, flush=True))
    finally:
        core.shutdown()
    return 0


def cmd_replay(args) -> None:
    sys.exit(main_from_namespace(args))


def main_from_namespace(args) -> int:
    core = make_core(args)
    try:
        replay(core, sys.stdin, args.out, say=lambda s: print(s, flush=True))
    finally:
        core.shutdown()
    return 0


if __name__ == "__main__":
    sys.exit(main())
