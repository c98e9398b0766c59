"""Batch generation over a .jsonl file:
``python -m torchllms_amd.inference.generate --input_path in.jsonl --output_path out.jsonl --provider_kwargs '{"ckpt_paths": "DIR"}'``.

Options keep the reference's names and meanings (reference: torchllms/inference/generate.py:10-62).
Every input line holds ``messages`` (a conversation, which is extended by the assistant's answer),
``prompt`` (a text, answered in ``completion``) or ``prompt_token_ids`` (answered in
``completion_token_ids``).  The only provider is this engine.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def parse_args(argv=None):
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--input_path", type=Path, required=True, help="Path of input .jsonl file.")
    p.add_argument("--output_path", type=Path, required=True, help="Path of output .jsonl file.")
    p.add_argument("--provider", type=str, default="torchllms", help="Model provider (only 'torchllms')")
    p.add_argument("--provider_kwargs", type=json.loads, default={}, help="JSON-encoded kwargs for LLM(...)")
    p.add_argument("--generate_kwargs", type=json.loads, default={}, help="JSON-encoded kwargs for LLM.generate")
    return p.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.provider != "torchllms":
        raise SystemExit(f"provider {args.provider!r} is not available; this engine offers 'torchllms' only")
    from .llm import LLM

    with open(args.input_path) as f:
        inputs = [json.loads(line) for line in f if line.strip()]
    if not inputs:
        raise SystemExit(f"{args.input_path} holds no records")
    llm = LLM(**args.provider_kwargs)
    if "messages" in inputs[0]:
        results = llm.generate(conversations=[r["messages"] for r in inputs], **args.generate_kwargs)
        for rec, res in zip(inputs, results):
            rec["messages"] = rec["messages"] + [{"role": "assistant", "content": res.text}]
    elif "prompt" in inputs[0]:
        results = llm.generate(prompts=[r["prompt"] for r in inputs], **args.generate_kwargs)
        for rec, res in zip(inputs, results):
            rec["completion"] = res.text
    else:
        results = llm.generate(prompt_token_ids=[r["prompt_token_ids"] for r in inputs], **args.generate_kwargs)
        for rec, res in zip(inputs, results):
            rec["completion_token_ids"] = res.token_ids
            rec["stop_reason"] = res.stop_reason
    args.output_path.parent.mkdir(parents=True, exist_ok=True)
    with open(args.output_path, "w") as f:
        for rec in inputs:
            f.write(json.dumps(rec) + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
