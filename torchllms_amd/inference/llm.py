"""``LLM``: load a model folder and generate from prompts, conversations or token ids.

The constructor and ``generate`` keep the reference's argument names and meanings where it has
them (reference: torchllms/inference/llm.py:95-109 constructor, 693-760 and 1076-1152 generate,
63-77 ``GenerationResult``).  Behind them sits this engine's continuous-batching scheduler in
place of the reference's one-prompt-at-a-time loop and static batches, so ``batched`` and
``batch_size`` are accepted and only bound how many requests run at once.
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, List, Optional, Sequence, Union

from ..messages.templates import ChatTemplate, FileTokenizer, get_template, tokenize_conversation
from ..sampling.params import SamplingParams


@dataclass
class GenerationResult:
    """``token_ids`` includes the stop token when generation stopped on one; ``text`` is decoded
    without special tokens; ``stop_reason`` is the stop token id, or None when the token budget
    or the context length ended generation (reference: llm.py:63-77)."""

    text: str
    token_ids: List[int]
    stop_reason: Optional[int]


class GenerationLoop:
    """Drives scheduler, step function and sampler until every request is done.  It needs an
    object with ``step(entries) -> logits`` and ``cache``, and a sampler
    ``(logits, params, steps) -> token ids``; nothing else."""

    def __init__(self, engine, sampler, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 prefill_chunk: Optional[int] = None, look_ahead: bool = True):
        from ..engine.scheduler import Scheduler

        self.engine = engine
        self.sampler = sampler
        self.look_ahead = look_ahead
        self.stats = {"prepared_steps": 0, "launched_ahead": 0}
        self.launch_ahead = look_ahead  # (a switch of its own for measurements)
        self._host_tokens = self._home = None
        self.scheduler = Scheduler(engine.cache, max_num_seqs, max_num_batched_tokens, max_model_len, prefill_chunk)

    def run(self, prompts: Sequence[Sequence[int]], params: Sequence[SamplingParams], on_step=None):
        """Generate for every prompt; returns the finished ``Request`` objects in input order.

        While the GPU runs a decode step, an engine that can (``prepare_decode``) prepares the next
        one for the case that the same requests decode again; the scheduler still decides every
        step, and the preparation is used only when its plan is that case.

        An engine that can (``step_prepared_on_device``) is then given the prepared step at once,
        with the sampled tokens still on the device, and the host reads them while that step runs:
        the GPU does not wait for the host between two decode steps.  This is done only where no
        request can reach its token budget with the sampled token, so the step is wrong only for a
        request that ends on a stop token: its row is dropped, the other rows are the step that
        the scheduler would have planned for them (one token each, pages taken by the
        preparation).  A step launched ahead is not put before the scheduler, so it is launched
        only while the scheduler could admit nobody anyway unless a request ends (nobody waits, or
        no seat is free, or pages are short and no layer gives pages back while it decodes): a
        request that waits is then admitted one step later than it would have been only when a
        request ended on the token that the step ahead was fed."""
        from ..engine.scheduler import ScheduledEntry, StepPlan

        sched = self.scheduler
        requests = [sched.add(("gen", id(self), i), p, sp) for i, (p, sp) in enumerate(zip(prompts, params))]
        prepare = getattr(self.engine, "prepare_decode", None) if self.look_ahead else None
        launch = getattr(self.sampler, "launch", None)
        launch_ahead = getattr(self.engine, "step_prepared_on_device", None) if self.look_ahead and self.launch_ahead else None
        prepared = None
        ahead = None  # (plan, logits) of a step that is already queued
        try:
            while sched.has_work:
                if ahead is not None:
                    plan, logits = ahead
                    ahead = None
                else:
                    plan = sched.schedule()
                    entries = plan.step_entries()
                    logits = None
                    if prepared is not None:
                        logits = self.engine.step_prepared(prepared, entries)  # None: it is another step
                        self.stats["prepared_steps"] += logits is not None
                    if logits is None:
                        logits = self.engine.step(entries)
                prepared = None
                sampling = [e.request for e in plan.entries if e.samples]
                counters = [len(r.output) for r in sampling]
                next_logits = None
                if prepare is not None and launch is not None and _decodes_on(plan):
                    prepared = prepare()  # the GPU is busy with the step meanwhile
                    go_ahead = prepared is not None and launch_ahead is not None and not sched.may_admit_before_a_request_ends()
                    # a step that is launched ahead gets its tokens where it reads them, straight from the sampling kernel
                    section = getattr(prepared, "token_section", None) if go_ahead else None
                    if section is not None:
                        pending = launch(logits, [r.params for r in sampling], counters, out=section())
                    else:
                        pending = launch(logits, [r.params for r in sampling], counters)
                    arriving = self._send_home(pending) if launch_ahead is not None else None
                    if go_ahead:
                        next_logits = launch_ahead(prepared, [e.request.rid for e in plan.entries], pending)
                    if next_logits is not None:
                        prepared = None  # used
                        self.stats["prepared_steps"] += 1
                        self.stats["launched_ahead"] += 1
                    tokens = self._arrived(arriving, pending.numel()) if arriving is not None else pending.tolist()
                else:
                    tokens = self.sampler(logits, [r.params for r in sampling], counters)
                sched.update(plan, tokens)
                if next_logits is not None:
                    # the step that is running: one token for every request that is still there
                    rows = [i for i, e in enumerate(plan.entries) if not e.request.finished]
                    if rows:
                        if len(rows) < len(plan.entries):
                            next_logits = next_logits[rows]
                        going_on = [plan.entries[i].request for i in rows]
                        ahead = (StepPlan(entries=[ScheduledEntry(r, [r.last_token], True) for r in going_on]), next_logits)
                if on_step is not None:
                    on_step(plan)
        except BaseException:
            # whatever happens, give pages and slots back (reference: llm.py:602-617)
            for r in requests:
                if not r.finished:
                    sched.abort(r)
            raise
        return requests

    def _send_home(self, pending):
        """Queue the copy of the sampled token ids to pinned host memory right behind the sampling,
        on the same stream, before anything else is queued: it is done as soon as the sampling
        is, whatever follows it.  (A copy on a stream of its own, waiting for an event behind the
        sampling, made every kernel of the step that ran meanwhile slower: a queue that waits is
        polled.)  Returns the event behind the copy."""
        import torch

        n = pending.numel()
        if not pending.is_cuda:  # an engine on the host (the tests' fake ones): nothing travels
            self._host_tokens = pending
            return _ARRIVED
        if self._host_tokens is None or self._host_tokens.numel() < n or not self._host_tokens.is_pinned():
            self._host_tokens = torch.empty((max(n, 64),), dtype=torch.int32, pin_memory=True)
            self._home = torch.cuda.Event()
        self._host_tokens[:n].copy_(pending, non_blocking=True)
        self._home.record()
        return self._home

    def _arrived(self, event, n: int) -> list:
        event.synchronize()
        return self._host_tokens[:n].tolist()


class _Arrived:
    def synchronize(self) -> None:
        pass


_ARRIVED = _Arrived()


def _decodes_on(plan) -> bool:
    """Is the plan a decode step after which every request surely decodes again (none reaches its
    token budget with this step's token; a stop token may still end one)?"""
    return bool(plan.entries) and all(
        len(e.tokens) == 1 and e.samples and len(e.request.output) + 1 < e.request.budget for e in plan.entries
    )


class LLM:
    def __init__(
        self,
        ckpt_paths: Union[str, Path, Sequence[Union[str, Path]]],
        template_config: Optional[str] = None,
        eos_ids: Optional[List[int]] = None,
        max_len: int = 4096,
        max_bsz: int = 4,
        device: str = "cuda",
        precision: Optional[str] = "bfloat16",
        model_kwargs: Optional[Dict[str, Any]] = None,
        batched: bool = True,
        page_size: int = 16,
        kv_memory_gb: Optional[float] = None,
        num_pages: Optional[int] = None,
        kv_memory_fraction: Optional[float] = None,
        max_num_batched_tokens: int = 2048,
        tokenizer=None,
        seed: int = 0,
        look_ahead: bool = True,
        kernel_table=None,
        random_weights: bool = False,
    ):
        """``ckpt_paths``: the model folder (config.json + safetensors), or a list whose first
        entry is that folder or a file in it.  ``precision``: "bfloat16" or "float32"; None takes
        config.json's ``torch_dtype``.  ``max_len`` bounds prompt + generated tokens of a request (as does the model's own maximum of positions),
        ``max_bsz`` the requests running at once.  ``model_kwargs`` may override ``max_seq_len``
        (reference: throughput_bench.py:1057-1060).  ``look_ahead``: prepare the next decode step
        while the GPU runs the current one (the tokens are the same either way).  ``kernel_table``:
        a saved table of matrix-product kernel choices (``Engine.kernel_table``), so that bfloat16
        results repeat from process to process.  ``random_weights``: the folder needs a config.json
        only (and a tokenizer.json for text); the weights are drawn from ``seed`` as
        ``weights.write_model_folder`` would write them."""
        from ..engine.engine import Engine
        from ..sampling.sampler import Sampler

        first = ckpt_paths if isinstance(ckpt_paths, (str, Path)) else list(ckpt_paths)[0]
        folder = Path(first)
        if folder.is_file():
            folder = folder.parent
        self.folder = folder
        if device == "cuda":
            device = "cuda:0"
        model_kwargs = dict(model_kwargs or {})
        if precision is None:
            import json

            with open(folder / "config.json") as f:
                precision = json.load(f).get("torch_dtype", "bfloat16")
        if "max_seq_len" in model_kwargs:
            max_len = min(max_len, int(model_kwargs.pop("max_seq_len")))
        if model_kwargs:
            raise ValueError(f"unknown model_kwargs {sorted(model_kwargs)}")
        engine_kw = dict(
            dtype=precision, device=device, page_size=page_size, num_pages=num_pages, kv_memory_gb=kv_memory_gb,
            kv_memory_fraction=kv_memory_fraction, max_seqs=max_bsz, max_model_len=max_len, kernel_table=kernel_table,
        )
        from ..config.registry import load_config

        arch, config = load_config(folder)
        # ``max_len`` is a bound, and so is the model's own maximum of positions
        engine_kw["max_model_len"] = min(max_len, arch.model_spec(config).max_positions)
        if random_weights:
            self.engine = Engine.from_random(config, seed=seed, arch=arch, **engine_kw)
        else:
            self.engine = Engine.from_folder(folder, **engine_kw)
        self.max_len = self.engine.max_model_len
        self.max_bsz = max_bsz
        self.batched = batched
        self.device = device
        self.seed = seed
        self.look_ahead = look_ahead
        self.max_num_batched_tokens = max_num_batched_tokens
        self.template: Optional[ChatTemplate] = get_template(template_config)
        if tokenizer is None and (folder / "tokenizer.json").is_file():
            tokenizer = FileTokenizer(folder / "tokenizer.json")
        self.tokenizer = tokenizer
        if self.template is not None and self.template.stop_token_ids:
            eos_ids = list(self.template.stop_token_ids)  # reference: llm.py:188-189
        if eos_ids is None:
            eos_ids = self.engine.arch.default_stop_token_ids(self.engine.config)
        self.eos_ids = list(eos_ids)
        self.sampler = Sampler()

    # ------------------------------------------------------------------ text <-> ids
    def _need_tokenizer(self):
        if self.tokenizer is None:
            raise ValueError("this model folder has no tokenizer.json: pass prompt_token_ids, or a tokenizer to LLM()")
        return self.tokenizer

    def tokenize_conversation(self, conversation) -> List[int]:
        tok = self._need_tokenizer()
        if self.template is None:
            raise ValueError("conversations need a template_config (for instance 'llama3_instruct')")
        return tokenize_conversation(conversation, tok, self.template, add_generation_prompt=True)

    # ------------------------------------------------------------------ generation
    def generate(
        self,
        prompts: Optional[List[str]] = None,
        conversations: Optional[List[List[Dict[str, str]]]] = None,
        temperature: float = 0.0,
        max_new_tokens: Optional[int] = None,
        batch_size: int = 0,
        disable_tqdm: bool = True,
        prompt_token_ids: Optional[List[List[int]]] = None,
        top_k: Optional[int] = None,
        stop_token_ids: Optional[Sequence[int]] = None,
        seed: Optional[int] = None,
    ) -> List[GenerationResult]:
        """Exactly one of ``prompts`` (texts, encoded without added special tokens),
        ``conversations`` (lists of role/content messages) and ``prompt_token_ids``.  Results come
        back in input order.  ``batch_size`` > 0 bounds the requests running at once below
        ``max_bsz``.  Request i is sampled with seed ``seed + i``."""
        given = [x is not None for x in (prompts, conversations, prompt_token_ids)]
        if sum(given) != 1:
            raise ValueError("give exactly one of prompts, conversations, prompt_token_ids")
        if conversations is not None:
            ids = [self.tokenize_conversation(c) for c in conversations]
        elif prompts is not None:
            tok = self._need_tokenizer()
            ids = [tok.encode(p) for p in prompts]
        else:
            ids = [list(p) for p in prompt_token_ids]
        stops = tuple(self.eos_ids if stop_token_ids is None else stop_token_ids)
        base = self.seed if seed is None else seed
        params = [
            SamplingParams(temperature=temperature, top_k=top_k, max_new_tokens=max_new_tokens, stop_token_ids=stops, seed=base + i)
            for i in range(len(ids))
        ]
        live = self.max_bsz if not batch_size else min(batch_size, self.max_bsz)
        if not self.batched:
            live = 1
        loop = GenerationLoop(self.engine, self.sampler, live, self.max_num_batched_tokens, self.max_len, look_ahead=self.look_ahead)
        finished = loop.run(ids, params)
        self.last_stats = dict(loop.scheduler.stats, **loop.stats)
        out = []
        for r in finished:
            text = self.tokenizer.decode(r.output) if self.tokenizer is not None else ""
            out.append(GenerationResult(text=text, token_ids=list(r.output), stop_reason=r.stop_reason))
        return out
