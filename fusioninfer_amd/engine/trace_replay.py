"""Replay a recorded step schedule through the engine and write logits.

    python -m fusioninfer_amd.engine.trace_replay --model DIR \\
        --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object per line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": []}

Every line is ONE engine step (LLMEngine.forced_step): all entries run as
one batch from the cache and state earlier steps left; ``want`` indexes
the entry's tokens whose logits are written to ``<out>/<step>.f32``
(little-endian fp32, [wanted, vocab], in the order of entries and want);
``end`` releases requests. After each step the line ``done <step>`` is
printed. The cache pool holds ``--max-tokens`` tokens and the state pool
``--max-seqs`` sequences, so pages and slots are recycled.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def parse_args(argv=None):
    p = argparse.ArgumentParser("fusioninfer-amd trace replay")
    p.add_argument("--model", required=True,
                   help="directory with config.json and model.safetensors")
    p.add_argument("--dtype", choices=["bfloat16", "float32"],
                   default="bfloat16")
    p.add_argument("--out", required=True)
    p.add_argument("--max-tokens", type=int, required=True,
                   help="cache pool size in tokens")
    p.add_argument("--max-seqs", type=int, default=4,
                   help="live requests (state slots)")
    p.add_argument("--enforce-eager", action="store_true",
                   help="no hipGraph capture for all-decode steps")
    p.add_argument("--device", default=None)
    return p.parse_args(argv)


def build_engine(args):
    import torch

    from fusioninfer_amd.config import (
        CacheConfig,
        EngineConfig,
        SchedulerConfig,
    )
    from fusioninfer_amd.engine.llm_engine import LLMEngine
    from fusioninfer_amd.models.registry import get_model_config

    mc = get_model_config(args.model)
    if mc.architecture == "transformer" and args.dtype != "bfloat16":
        # the built-in transformer family is bf16-only
        sys.stderr.write("float32 is not available for this model family\n")
        sys.exit(3)
    mc.dtype = args.dtype
    if args.dtype == "float32":
        # true fp32 matrix products: no reduced-precision GEMM modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    cache = CacheConfig(enable_prefix_caching=False)
    bs = cache.block_size
    cache.num_gpu_blocks = (args.max_tokens + bs - 1) // bs
    cfg = EngineConfig(
        model=mc,
        cache=cache,
        scheduler=SchedulerConfig(
            max_num_seqs=args.max_seqs,
            max_num_batched_tokens=max(args.max_tokens, 1),
            max_model_len=max(args.max_tokens, 1),
        ),
        enforce_eager=args.enforce_eager,
        num_state_slots=args.max_seqs,
    )
    device = args.device or ("cuda:0" if torch.cuda.is_available() else "cpu")
    return LLMEngine(cfg, device=device)


def main(argv=None) -> int:
    args = parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    engine = build_engine(args)
    import numpy as np

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or [])
                   for e in step.get("entries", [])]
        logits = engine.forced_step(entries, step.get("end") or [])
        if logits is not None and logits.shape[0] > 0:
            arr = np.ascontiguousarray(
                logits.detach().cpu().numpy().astype("<f4"))
            tmp = os.path.join(args.out, ".%s.tmp" % step["step"])
            with open(tmp, "wb") as f:
                f.write(arr.tobytes())
            os.replace(tmp, os.path.join(args.out, "%s.f32" % step["step"]))
        sys.stdout.write("done %s\n" % step["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
