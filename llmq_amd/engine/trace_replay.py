"""Replay a token trace through the engine and write logits.

A trace is a stream of steps on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Each entry gives a request its next tokens (teacher-forced — nothing is
sampled) and the positions among them whose logits are wanted; ``end`` names
the requests that are finished after the step. All entries of a step run as
ONE engine batch (LLMEngine.replay_step): the scheduler's block and state-slot
allocators, the model runner's prefill / decode / mixed paths and the HIP
kernels are the ones generation uses. For a step with wanted positions the
logits are written to OUT/<step>.f32 (little-endian fp32 [wanted, vocab], in
entry order); after every step ``done <step>`` is printed.

The KV pool is sized for --max-tokens live tokens (rounded up to whole
blocks) and four live requests, so blocks and state slots are reused across
the trace.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List, Optional

MAX_LIVE_REQUESTS = 4


def build_engine(model: str, dtype: str, max_tokens: int):
    import torch

    from llmq_amd.engine.config import EngineConfig
    from llmq_amd.engine.engine import LLMEngine
    from llmq_amd.engine.model_specs import resolve_spec
    from llmq_amd.engine.models import model_class_for

    if torch.cuda.is_available():
        # compile what this model family runs on, if no built library exists
        from llmq_amd.ops.build import ensure

        spec = resolve_spec(model)
        for group in getattr(model_class_for(spec), "ext_groups", ("main",)):
            ensure(group)
        # fp32 means fp32: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    block = 16
    cfg = EngineConfig(
        model=model, dtype=dtype, max_num_seqs=MAX_LIVE_REQUESTS,
        max_model_len=max(max_tokens, block), kv_block_size=block,
        num_kv_blocks=(max_tokens + block - 1) // block,
        max_prefill_tokens=max(max_tokens, block),
    )
    return LLMEngine(cfg)


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    import logging

    logging.basicConfig(stream=sys.stderr, level=logging.WARNING)
    engine = build_engine(args.model, args.dtype, args.max_tokens)
    import numpy as np

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = engine.replay_step(step.get("entries") or [], step.get("end") or [])
        if logits.shape[0]:
            arr = np.ascontiguousarray(logits.detach().float().cpu().numpy().astype("<f4"))
            tmp = os.path.join(args.out, f".{step['step']}.part")
            with open(tmp, "wb") as fh:
                fh.write(arr.tobytes())
            os.replace(tmp, os.path.join(args.out, f"{step['step']}.f32"))
        sys.stdout.write(f"done {step['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
