"""Interactive chat: ``python -m torchllms_amd.inference.chat --ckpt_paths DIR --template_config llama3_instruct``.

Options and the dialogue keep the reference's names and meanings (reference:
torchllms/inference/chat.py:16-91): a ``[system]:`` line first (may be empty), then ``[user]:``
turns answered after ``[assistant]:``; ``!!reset`` starts over.  Each option also answers to a
dashed spelling (``--model``, ``--dtype``, ``--max-new-tokens``, ``--max-model-len``); what the
reference lacks and this engine adds: ``--random-weights`` (the folder then needs config.json and
tokenizer.json only; weights come from ``--seed``), ``--page_size``, ``--kv_memory_gb``, ``--seed``.
"""

from __future__ import annotations

import argparse
import json
import sys

YELLOW, NORMAL = "\033[33m", "\033[0m"


def parse_args(argv=None):
    p = argparse.ArgumentParser(description="Interactive chat with a model folder on one AMD GPU.")
    p.add_argument("--ckpt_paths", "--model", nargs="+", required=True, dest="ckpt_paths",
                   help="Model folder (config.json, safetensors, tokenizer.json); further paths are ignored.")
    p.add_argument("--template_config", "--template-config", type=str, default="llama3_instruct", help="Name of the chat template.")
    p.add_argument("--max_new_tokens", "--max-new-tokens", type=int, default=200, help="Maximum number of new tokens.")
    p.add_argument("--temperature", type=float, default=0.0, help="Temperature for sampling.")
    p.add_argument("--device", type=str, default="cuda", help="Device to use")
    p.add_argument("--precision", "--dtype", type=str, default=None, dest="precision", help="Precision to use, otherwise the checkpoint's")
    p.add_argument("--model_kwargs", "--model-kwargs", type=json.loads, default={}, help="JSON: further model options (max_seq_len)")
    p.add_argument("--max_len", "--max-model-len", type=int, default=4096, dest="max_len", help="Longest prompt plus answer, in tokens")
    p.add_argument("--page_size", "--page-size", type=int, default=16)
    p.add_argument("--kv_memory_gb", "--kv-memory-gb", type=float, default=None)
    p.add_argument("--seed", type=int, default=0, help="Seed of sampling (and of --random-weights)")
    p.add_argument("--random-weights", "--random_weights", action="store_true",
                   help="Draw the weights from --seed instead of reading safetensors (the folder needs config.json only)")
    return p.parse_args(argv)


def _ask(label: str) -> str:
    return input(f"{YELLOW}[{label}]: {NORMAL}").strip()


def _start_conversation():
    conversation = []
    system_message = _ask("system")
    if system_message:
        conversation.append({"role": "system", "content": system_message})
    return conversation


def main(argv=None) -> int:
    args = parse_args(argv)
    from .llm import LLM

    print("Loading model and tokenizer...")
    llm = LLM(
        ckpt_paths=args.ckpt_paths, template_config=args.template_config, device=args.device,
        precision=args.precision, model_kwargs=args.model_kwargs, max_len=args.max_len, max_bsz=1,
        page_size=args.page_size, kv_memory_gb=args.kv_memory_gb, seed=args.seed, random_weights=args.random_weights,
    )
    try:
        conversation = _start_conversation()
        while True:
            content = _ask("user")
            if content == "!!reset":
                conversation = _start_conversation()
                continue
            conversation.append({"role": "user", "content": content})
            result = llm.generate(conversations=[conversation], max_new_tokens=args.max_new_tokens,
                                  temperature=args.temperature)[0]
            conversation.append({"role": "assistant", "content": result.text})
            print(f"{YELLOW}[assistant]: {NORMAL}{result.text}")
    except (EOFError, KeyboardInterrupt):
        print()
        return 0


if __name__ == "__main__":
    sys.exit(main())
