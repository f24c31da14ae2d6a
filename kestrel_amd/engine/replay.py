"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: every step goes
through ``ModelRunner.step``, the function generation uses.

Input: one JSON object a line on standard input,
``{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}``.
All entries of a step are one batch. For a step in which something is wanted the logits
at the wanted places are written to ``<out>/<step>.f32`` as little-endian float32
``[wanted, vocab]`` in the order of the entries and of ``want``. After every step a line
``done <step>`` is printed and flushed. Requests named in ``end`` give back what they
hold after the step.

Two optional keys of an entry go beyond token ids: ``embeds`` (rows for the places whose
token id is -1) and ``bidirectional`` (position ranges ``[lo, hi)`` that see each other both
ways and must lie inside the portion).
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Dict

import numpy as np


def parse_args(argv=None):
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder the logits are written to")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to 64)")
    parser.add_argument("--page-size", type=int, default=16, help="tokens per cache page (must divide 64)")
    parser.add_argument("--max-requests", type=int, default=64, help="most requests live at a time")
    parser.add_argument("--device", default="cuda:0")
    return parser.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.max_tokens <= 0:
        print("trace_run: --max-tokens must be positive", file=sys.stderr)
        return 2
    if args.page_size <= 0 or 64 % args.page_size:
        print("trace_run: --page-size must divide 64", file=sys.stderr)
        return 2
    import torch

    from ..config.runtime import parse_dtype
    from .loading import load_model, make_runner
    from .step import StepEntry

    device = torch.device(args.device)
    dtype = parse_dtype(args.dtype)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    net = load_model(args.model, dtype, device)
    n_pages = -(-args.max_tokens // args.page_size)
    runner = make_runner(net, args.page_size, n_pages, args.max_requests,
                         max_tokens_per_step=max(args.max_tokens, 64))
    slots: Dict[str, int] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            name = str(item["id"])
            if name not in slots:
                slots[name] = runner.admit()
            embeds = item.get("embeds")
            entries.append(StepEntry(
                slot=slots[name], tokens=item["tokens"], want=item.get("want", []),
                embeds=None if embeds is None else torch.tensor(embeds, dtype=torch.float32),
                bidirectional=[tuple(b) for b in item.get("bidirectional", [])]))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                np.ascontiguousarray(logits.cpu().numpy(), dtype="<f4").tofile(out_dir / f"{step}.f32")
        for name in record.get("end", []):
            name = str(name)
            if name in slots:
                runner.release(slots.pop(name))
        print(f"done {step}", flush=True)
    torch.cuda.synchronize(device)
    return 0


if __name__ == "__main__":
    sys.exit(main())
