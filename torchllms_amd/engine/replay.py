"""Trace replay: feeds given token ids through the engine step by step and writes logits.

It samples nothing and owns no model code: it drives ``Engine.step``, the same step function,
cache and kernels that generation uses.  The reference has no such tool; its nearest relative is
the logit-capturing forward hook of its validator (reference:
torchllms/inference/validate_qwen3.py:203-264).

Input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` receives the logits at the wanted
places (order of the entries, then of ``want``) as little-endian float32 [wanted, vocab].  After
every step the line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path



def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder the logits files are written to")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (each request rounded up to 64)")
    p.add_argument("--page-size", type=int, default=16, help="tokens per cache page (default 16)")
    p.add_argument("--max-seqs", type=int, default=8, help="request slots (default 8)")
    p.add_argument("--kernel-table", default=None,
                   help="JSON file of matrix-product kernel choices (bfloat16): read if it exists, so that this run uses "
                        "the kernels of the run that wrote it and rounds as that run did; else written after the "
                        "choices have been measured")
    p.add_argument("--device", default="cuda:0")
    return p


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)

    print("[trace_run] loading kernels (compiles on first use)", file=sys.stderr, flush=True)
    from ..kernels import lib

    lib.core()
    from .engine import Engine
    from .layout import StepEntry

    if args.page_size <= 0:
        raise SystemExit("--page-size must be positive")
    # --max-tokens counts every request rounded up to 64 tokens; with pages that neither divide 64
    # nor are a multiple of it a request's last page may reach beyond that, so each slot gets one more
    num_pages = max(-(-args.max_tokens // args.page_size), 1)
    if 64 % args.page_size and args.page_size % 64:
        num_pages += args.max_seqs
    print(f"[trace_run] loading {args.model} as {args.dtype}; pool of {num_pages} pages of {args.page_size} tokens",
          file=sys.stderr, flush=True)
    table = Path(args.kernel_table) if args.kernel_table else None
    engine = Engine.from_folder(
        args.model, dtype=args.dtype, device=args.device, page_size=args.page_size, num_pages=num_pages,
        max_seqs=args.max_seqs, kernel_table=str(table) if table is not None and table.is_file() else None,
    )
    if args.dtype == "bfloat16":
        used = engine.kernel_table()
        if table is not None and not table.is_file():
            with open(table, "w") as f:
                json.dump(used, f, indent=1)
        print(f"[trace_run] matrix-product kernels: {json.dumps(used)}", file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if not engine.cache.has(rid):
                engine.admit(rid)
            entries.append(StepEntry(rid=rid, tokens=list(e["tokens"]), want=list(e.get("want", []))))
        logits = engine.step(entries)
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            arr.tofile(out_dir / f"{step}.f32")
        for rid in rec.get("end", []):
            if engine.cache.has(rid):
                engine.free(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
