"""Batch generation over a .jsonl file:
``python -m torchllms_amd.inference.generate --input_path in.jsonl --output_path out.jsonl --provider_kwargs '{"ckpt_paths": "DIR"}'``.

Options keep the reference's names and meanings (reference: torchllms/inference/generate.py:10-62).
Every input line holds ``messages`` (a conversation, which is extended by the assistant's answer),
``prompt`` (a text, answered in ``completion``) or ``prompt_token_ids`` (answered in
``completion_token_ids``).  The only provider is this engine.

Without a file: ``--model DIR --prompt "text"`` or ``--prompt-ids 5 17 3`` answer one prompt and print
the completion (text, or token ids) on standard output; ``--random-weights --seed N`` draws the weights
instead of reading them, ``--dtype``, ``--max-new-tokens``, ``--temperature`` as in the chat program.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def parse_args(argv=None):
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--input_path", "--input-path", type=Path, default=None, help="Path of input .jsonl file.")
    p.add_argument("--output_path", "--output-path", type=Path, default=None, help="Path of output .jsonl file.")
    p.add_argument("--provider", type=str, default="torchllms", help="Model provider (only 'torchllms')")
    p.add_argument("--provider_kwargs", "--provider-kwargs", type=json.loads, default={}, help="JSON-encoded kwargs for LLM(...)")
    p.add_argument("--generate_kwargs", "--generate-kwargs", type=json.loads, default={}, help="JSON-encoded kwargs for LLM.generate")
    p.add_argument("--prompt", type=str, default=None, help="One prompt as text, instead of --input_path")
    p.add_argument("--prompt-ids", "--prompt_ids", type=int, nargs="+", default=None, help="One prompt as token ids, instead of --input_path")
    p.add_argument("--model", "--ckpt_paths", type=str, default=None, dest="model", help="Model folder (short for provider_kwargs.ckpt_paths)")
    p.add_argument("--dtype", "--precision", type=str, default=None, dest="dtype")
    p.add_argument("--random-weights", "--random_weights", action="store_true")
    p.add_argument("--seed", type=int, default=None)
    p.add_argument("--template_config", "--template-config", type=str, default=None)
    p.add_argument("--max-new-tokens", "--max_new_tokens", type=int, default=None)
    p.add_argument("--temperature", type=float, default=None)
    args = p.parse_args(argv)
    given = [args.input_path is not None, args.prompt is not None, args.prompt_ids is not None]
    if sum(given) != 1:
        p.error("give exactly one of --input_path, --prompt and --prompt-ids")
    if args.input_path is not None and args.output_path is None:
        p.error("--input_path needs --output_path")
    # the short options end up where the JSON options put them
    for key, value in (("ckpt_paths", args.model), ("precision", args.dtype), ("seed", args.seed), ("template_config", args.template_config)):
        if value is not None:
            args.provider_kwargs[key] = value
    if args.random_weights:
        args.provider_kwargs["random_weights"] = True
    for key, value in (("max_new_tokens", args.max_new_tokens), ("temperature", args.temperature)):
        if value is not None:
            args.generate_kwargs[key] = value
    if "ckpt_paths" not in args.provider_kwargs:
        p.error("no model: give --model DIR or provider_kwargs with ckpt_paths")
    return args


def answer(llm, records, generate_kwargs):
    """Extend every record by the model's answer, in the field that fits its kind of prompt."""
    if "messages" in records[0]:
        results = llm.generate(conversations=[r["messages"] for r in records], **generate_kwargs)
        for rec, res in zip(records, results):
            rec["messages"] = rec["messages"] + [{"role": "assistant", "content": res.text}]
    elif "prompt" in records[0]:
        results = llm.generate(prompts=[r["prompt"] for r in records], **generate_kwargs)
        for rec, res in zip(records, results):
            rec["completion"] = res.text
    else:
        results = llm.generate(prompt_token_ids=[r["prompt_token_ids"] for r in records], **generate_kwargs)
        for rec, res in zip(records, results):
            rec["completion_token_ids"] = res.token_ids
            rec["stop_reason"] = res.stop_reason
    return records


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.provider != "torchllms":
        raise SystemExit(f"provider {args.provider!r} is not available; this engine offers 'torchllms' only")
    from .llm import LLM

    if args.input_path is not None:
        with open(args.input_path) as f:
            records = [json.loads(line) for line in f if line.strip()]
        if not records:
            raise SystemExit(f"{args.input_path} holds no records")
    elif args.prompt is not None:
        records = [{"prompt": args.prompt}]
    else:
        records = [{"prompt_token_ids": list(args.prompt_ids)}]
    llm = LLM(**args.provider_kwargs)
    answer(llm, records, args.generate_kwargs)
    if args.output_path is not None:
        args.output_path.parent.mkdir(parents=True, exist_ok=True)
        with open(args.output_path, "w") as f:
            for rec in records:
                f.write(json.dumps(rec) + "\n")
    if args.input_path is None:
        rec = records[0]
        print(rec["completion"] if "completion" in rec else " ".join(str(t) for t in rec["completion_token_ids"]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
