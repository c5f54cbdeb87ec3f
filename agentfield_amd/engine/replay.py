"""Trace replay: feed given token ids through a served model step by step
and write the logits at requested places.  Nothing is sampled.

The replay drives the serving engine itself — its model registry and weight
loading, page and state-slot allocation, packed-batch construction and
kernels (LLMEngine.open_request / feed_step / close_request) — so a trace
exercises exactly what generation runs.

Input, one JSON object per line on stdin:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": ["a"]}

`entries` lists, per live request, its next tokens and the offsets among
them whose logits are wanted; all entries of a step run as one batch.  A
request is admitted at its first entry and gives back its pages and state
slot when a step's `end` names it.  For a step with wanted rows the logits
are written to OUT/<step>.f32 (little-endian fp32, [wanted, vocab], entry
order); after every step `done <step>` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PAGE = 64
MAX_LIVE = 4


def build_engine(model_dir: str, dtype_name: str, max_tokens: int,
                 device: str | None = None, max_live: int = MAX_LIVE):
    import torch
    from ..models.registry import load_model
    from .engine import LLMEngine
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype_name]
    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    if dtype == torch.float32:
        # true fp32 matrix products
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    pages = (max_tokens + PAGE - 1) // PAGE
    model = load_model(model_dir, device=device, dtype=dtype,
                       max_position=pages * PAGE)
    # +1: page 0 is the engine's null page
    return LLMEngine(model.cfg, device=device, dtype=dtype, page_size=PAGE,
                     num_pages=pages + 1, max_num_seqs=max_live, model=model,
                     enable_graphs=False, caller_paced=True)


def run(engine, lines, out_dir: Path, emit=print) -> None:
    import numpy as np
    live: dict[str, object] = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = []
        for e in step.get("entries", []):
            seq = live.get(e["id"])
            if seq is None:
                seq = live[e["id"]] = engine.open_request()
            entries.append((seq, [int(t) for t in e["tokens"]],
                            [int(w) for w in e.get("want", [])]))
        logits = engine.feed_step(entries)
        if logits is not None:
            arr = logits.detach().to("cpu").contiguous().numpy()
            arr.astype("<f4", copy=False).tofile(
                str(out_dir / f"{step['step']}.f32"))
        for rid in step.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                engine.close_request(seq)
        emit(f"done {step['step']}")


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--model", required=True,
                    help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"],
                    default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time")
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)
    out = Path(a.out)
    out.mkdir(parents=True, exist_ok=True)
    engine = build_engine(a.model, a.dtype, a.max_tokens, a.device)
    run(engine, sys.stdin, out,
        emit=lambda s: (sys.stdout.write(s + "\n"), sys.stdout.flush()))
    return 0


if __name__ == "__main__":
    sys.exit(main())
