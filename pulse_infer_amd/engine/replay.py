"""The program behind ``bin/trace_run``: it drives ``ModelRunner`` with the tokens a trace gives."""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, List, Optional

PAGE_SIZE = 16
ROUND_TO = 64
MAX_LIVE = 4


def parse_args(argv: Optional[List[str]] = None) -> argparse.Namespace:
    p = argparse.ArgumentParser(prog="trace_run", description="Replay token ids step by step and write float32 logits.")
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"],
                   help="bfloat16: the kernels and precisions of serving; float32: everything in true 32-bit")
    p.add_argument("--out", required=True, help="folder that receives <step>.f32")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    p.add_argument("--page-size", type=int, default=PAGE_SIZE, help="tokens per cache page (divides 64)")
    p.add_argument("--device", default="cuda:0")
    return p.parse_args(argv)


def main(argv: Optional[List[str]] = None) -> int:
    args = parse_args(argv)
    if args.page_size <= 0 or ROUND_TO % args.page_size:
        print(f"trace_run: --page-size must divide {ROUND_TO}", file=sys.stderr)
        return 2
    if args.max_tokens <= 0:
        print("trace_run: --max-tokens must be positive", file=sys.stderr)
        return 2
    os.makedirs(args.out, exist_ok=True)

    import numpy as np
    import torch

    if not torch.cuda.is_available():
        print("trace_run: no GPU is visible; this engine has no CPU path", file=sys.stderr)
        return 3
    from ..models.factory import load_model
    from .runner import ModelRunner, StepEntry

    torch.backends.cuda.matmul.allow_tf32 = False
    _, model = load_model(args.model, mode=args.dtype, device=args.device)
    pool_tokens = (args.max_tokens + ROUND_TO - 1) // ROUND_TO * ROUND_TO
    runner = ModelRunner(model, page_size=args.page_size, num_pages=pool_tokens // args.page_size,
                         max_requests=max(MAX_LIVE, 8))
    held: Dict[str, int] = {}

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            rid = item["id"]
            tokens = [int(t) for t in item["tokens"]]
            if not runner.cache.has_request(rid):
                runner.add_request(rid)
                held[rid] = 0
            held[rid] += len(tokens)
            runner.reserve(rid, held[rid])
            entries.append(StepEntry(rid, tokens, [int(w) for w in item.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                data = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{step}.f32.tmp")
                data.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
            else:
                torch.cuda.synchronize()
        for rid in record.get("end", []):
            if runner.cache.has_request(rid):
                runner.free_request(rid)
            held.pop(rid, None)
        print(f"done {step}", flush=True)
    return 0
