"""The engine: a model, its cache and the one step function that everything else drives.

``Engine.step`` takes a batch of (request, its next tokens) — portions of prompts beside single
decoded tokens, cut anywhere —, runs exactly those tokens as one batch against the cache, and
returns the logits at the wanted places.  Generation, the scheduler and trace replay all go
through it.  The reference's counterpart is ``Transformer.forward`` with a ``PagedKVPool``
(reference: torchllms/models/networks.py:909-1049), which must be given *all* live rollouts in
claim order (networks.py:985-990); here any subset of the live requests may run, in any order.
"""

from __future__ import annotations

from typing import Dict, Hashable, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, OutOfPages, group_layers
from ..config.registry import ArchSpec, architecture_of, load_config
from ..parts.model import Model
from ..weights.loader import load_weights
from ..weights.random_init import random_tensor, random_tensors
from .context import upload
from .layout import StepEntry, StepLayout, build_step_layout

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "fp32": torch.float32, "bf16": torch.bfloat16}


def parse_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype must be float32 or bfloat16, got {dtype}")
        return dtype
    try:
        return DTYPES[str(dtype)]
    except KeyError:
        raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}") from None


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError(
            "this engine runs on an AMD GPU only (there is no CPU path); "
            f"asked for device {device}, torch.cuda.is_available()={torch.cuda.is_available()}"
        )
    return device


class PreparedDecode:
    """A decode step whose plan is made and uploaded but for its tokens (``Engine.prepare_decode``)."""

    __slots__ = ("rids", "wants", "previous", "layout", "graph", "epoch")

    def __init__(self, rids, wants, previous, layout, graph, epoch):
        self.rids, self.wants, self.previous, self.layout, self.graph, self.epoch = rids, wants, previous, layout, graph, epoch

    def token_section(self) -> torch.Tensor:
        """int32 [requests] on the device: where the step reads its token ids.  A sampling kernel may write
        them there; ``Engine.step_prepared_on_device`` given this tensor copies nothing."""
        return self.graph.token_section(len(self.rids))


class Engine:
    def __init__(
        self,
        arch: ArchSpec,
        config,
        tensors: Dict[str, torch.Tensor],
        dtype: torch.dtype,
        page_size: int = 16,
        num_pages: Optional[int] = None,
        kv_memory_gb: Optional[float] = None,
        kv_memory_fraction: Optional[float] = None,
        max_seqs: int = 8,
        max_model_len: Optional[int] = None,
        device="cuda:0",
        use_graphs: bool = True,
        tune_kernels: bool = True,
        kernel_table=None,
        beyond_max_positions: bool = False,
    ):
        """``tensors``: the model's tensors under the parts' own names, on ``device``.
        Pool size: room for ``num_pages`` pages of ``page_size`` tokens, else what ``kv_memory_gb``
        holds, else ``kv_memory_fraction`` of the device memory that is free once the weights are
        loaded, else room for ``max_seqs`` requests of ``max_model_len`` tokens (reference:
        networks.py:872-884); a group of layers with a page size of its own gets as many pages as
        hold the same number of tokens.

        Which bfloat16 matrix-product kernel serves a decode step is looked up in a table by shape,
        row count and use.  ``kernel_table`` (a dict as ``kernel_table()`` returns, or the path of a
        JSON file of one) fills the table first; ``tune_kernels`` then measures what the table does
        not hold yet.  Kernels differ in rounding, so two processes agree bit for bit in bfloat16
        only when they run from the same table; with ``tune_kernels=False`` and no table every shape
        follows a fixed rule of sizes (``ops.linear_choice``).

        ``max_model_len`` (default: the configuration's maximum of positions) may exceed that
        maximum only with ``beyond_max_positions``."""
        self.device = require_gpu(device)
        self.arch = arch
        self.config = config
        self.dtype = dtype
        self.spec = arch.model_spec(config)
        self.model = Model(self.spec)
        # a size that no kernel takes is refused here, not at the first step
        self.model.check_sizes(dtype)
        if page_size <= 0:
            raise ValueError(f"page_size must be positive, got {page_size}")
        self.model.bind(tensors)
        self.vocab_size = self.spec.vocab_size
        # the reference's table of rotation angles ends at the configuration's maximum and a longer
        # request fails there (reference: networks.py:325-327); angles are computed from positions
        # here, so a longer context would run, on positions the model never saw: only when asked
        if max_model_len is not None and max_model_len > self.spec.max_positions and not beyond_max_positions:
            raise ValueError(
                f"max_model_len={max_model_len} exceeds the {self.spec.max_positions} positions of the model's "
                "configuration; pass beyond_max_positions=True to run longer contexts all the same"
            )
        self.max_model_len = int(max_model_len or self.spec.max_positions)
        self.page_size = page_size
        from ..kernels import ops

        if kernel_table is not None:
            ops.load_kernel_table(kernel_table)
        if dtype == torch.bfloat16 and tune_kernels:
            # which matrix-product kernel serves decode steps best is measured, not guessed; before
            # the pool is sized, so that what the measurement borrows is free again for pages
            for (shape, use, out_dtype), group in self.model.linear_weights().items():
                ops.tune_linear(group, out_dtype or torch.bfloat16, use)
            torch.cuda.empty_cache()
        groups, states = group_layers(self.model.cache_needs())
        if isinstance(num_pages, dict):
            pages = dict(num_pages)
        else:
            if num_pages is not None:
                capacity = int(num_pages) * page_size
            else:
                per_token = CacheManager.bytes_per_token(groups, dtype)
                if kv_memory_gb is not None and per_token > 0:
                    capacity = int(kv_memory_gb * (1 << 30)) // per_token
                elif kv_memory_fraction is not None and per_token > 0:
                    if not 0.0 < kv_memory_fraction <= 1.0:
                        raise ValueError(f"kv_memory_fraction must lie in (0, 1], got {kv_memory_fraction}")
                    free_bytes, _ = torch.cuda.mem_get_info(self.device)
                    capacity = int(free_bytes * kv_memory_fraction) // per_token
                else:
                    capacity = max_seqs * (-(-self.max_model_len // page_size)) * page_size
            pages = CacheManager.pages_for_tokens(groups, page_size, max(capacity, 1))
        self.cache = CacheManager(groups, states, page_size, pages, max_seqs, dtype=dtype, device=self.device)
        self.steps_run = 0
        self.tokens_run = 0
        # the last step's plan when every row of it brought one token: (request ids, wanted places,
        # layout); a decode step that follows it with the same requests is planned from it
        self._last_decode = None
        # decode steps are replayed from HIP graphs when every part's launches are fixed by the
        # step's shape alone
        from .graphs import DecodeGraphs

        graph_safe = all(getattr(p, "graph_safe", False) for p in self.model.all_parts())
        self.graphs = DecodeGraphs(self.model, self.cache, self.device) if (use_graphs and graph_safe) else None

    def kernel_table(self) -> dict:
        """The table entries of this model's matrices (JSON-able): hand it to another engine, or
        save it with ``ops.save_kernel_table``, to run the same kernels in another process."""
        from ..kernels import ops

        shapes = {(shape, use) for (shape, use, _), group in self.model.linear_weights().items()}
        return ops.kernel_table(shapes)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        """A model folder holds ``config.json`` and safetensors; the architecture named in
        config.json picks the model."""
        device = require_gpu(device)
        dtype = parse_dtype(dtype)
        arch, config = load_config(folder)
        spec = arch.model_spec(config)
        model = Model(spec)
        model.check_sizes(dtype)  # before the weights are read: a refusal costs nothing
        expected = model.param_specs()
        ignore = model.ignorable_tensors()
        tensors = load_weights(folder, arch.weight_rules(config), expected, dtype, device=device, ignore_when_present=ignore)
        return cls._from_tensors(arch, config, tensors, dtype, device, kw)

    @classmethod
    def _from_tensors(cls, arch, config, tensors, dtype, device, kw) -> "Engine":
        engine = cls(arch, config, tensors, dtype, device=device, **kw)
        # parts that fuse matrices (q|k|v, gate|up) hold copies; the separate ones go with this dictionary,
        # and their memory goes back to the device instead of staying in torch's cache
        tensors.clear()
        torch.cuda.empty_cache()
        return engine

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", norm_jitter: float = 0.0,
                    draw_on_device: bool = False, arch: Optional[ArchSpec] = None, **kw) -> "Engine":
        """Random weights without a folder: same values as ``write_model_folder`` with this seed
        when drawn on the CPU; ``draw_on_device`` draws on the GPU instead (large models)."""
        device = require_gpu(device)
        dtype = parse_dtype(dtype)
        arch = arch or architecture_of(config)
        model = Model(arch.model_spec(config))
        model.check_sizes(dtype)
        expected = model.param_specs()
        if draw_on_device:
            tensors = random_tensors(expected, seed, dtype, norm_jitter, device=device)
        else:
            # one tensor at a time (a few at once, each with a generator of its own), so that the host never
            # holds more than a few tensors of the model in 32-bit
            from concurrent.futures import ThreadPoolExecutor

            def draw(item):
                name, spec = item
                return name, random_tensor(name, spec, seed, torch.float32, norm_jitter).to(dtype).to(device)

            with ThreadPoolExecutor(max_workers=4) as pool:
                tensors = dict(pool.map(draw, expected.items()))
        return cls._from_tensors(arch, config, tensors, dtype, device, kw)

    # ------------------------------------------------------------------ requests
    def admit(self, rid: Hashable) -> int:
        return self.cache.admit(rid)

    def free(self, rid: Hashable) -> None:
        self.cache.free(rid)

    def num_tokens(self, rid: Hashable) -> int:
        return self.cache.num_tokens(rid)

    # ------------------------------------------------------------------ the step
    def _plan_next_decode(self, entries: Sequence[StepEntry]) -> Optional[StepLayout]:
        """The plan of a decode step that follows a decode step of the same requests, made from
        that step's plan: positions move on by one, a block table gains an entry where a page
        begins.  None when the step is anything else (the general planner then checks and says
        what is wrong with it)."""
        last = self._last_decode
        if last is None or len(entries) != len(last[0]):
            return None
        rids, wants, prev, epoch = last
        toks = []
        for e, rid, want in zip(entries, rids, wants):
            if e.rid != rid or len(e.tokens) != 1 or list(e.want) != want:
                return None
            toks.append(e.tokens[0])
        if min(toks) < 0 or max(toks) >= self.vocab_size:
            return None
        layout = self._next_decode_layout()
        if layout is not None:
            layout.tokens[:] = toks
        return layout

    def _next_decode_layout(self) -> Optional[StepLayout]:
        """What ``_plan_next_decode`` knows before it has seen the tokens: the plan of the next
        decode step of the last decode step's requests, with zeros for token ids.  Takes the pages
        that the step needs; None, with nothing taken, when it cannot be."""
        last = self._last_decode
        if last is None:
            return None
        rids, wants, prev, epoch = last
        cache = self.cache
        if epoch != cache.epoch:
            return None
        n = len(rids)
        held = prev.kv_lens.tolist()
        get = cache.get
        for rid, have in zip(rids, held):
            live = get(rid)
            if live is None or live.num_tokens != have:
                return None
        if max(held) + 1 > self.max_model_len:
            return None
        positions = prev.kv_lens.copy()  # the new token's position = tokens held so far
        # rows whose new token opens a page, per group; the others have room
        fresh = [(positions % page) == 0 for page in cache.page_sizes]
        opening = np.zeros(n, dtype=bool)
        for f in fresh:
            opening |= f
        opening = np.nonzero(opening)[0]
        if opening.size:
            need = [0] * len(cache.pools)
            for i in opening:  # (a page taken by an earlier preparation of this very step is not needed again)
                for g, pages in enumerate(cache.new_pages_needed(rids[i], 1)):
                    need[g] += pages
            if any(k > pool.free_count for k, pool in zip(need, cache.pools)):
                return None
            for i in opening:
                cache.extend(rids[i], 1)
        tables, slots = [], []
        for g, page in enumerate(cache.page_sizes):
            bt = prev.block_tables[g]
            sm = prev.slot_mappings[g] + 1
            if fresh[g].any():
                width = max(bt.shape[1], int(positions.max()) // page + 1)
                wider = np.full((n, width), -1, dtype=np.int32)
                wider[:, : bt.shape[1]] = bt
                bt = wider
                for i in np.nonzero(fresh[g])[0]:
                    blk = int(positions[i]) // page
                    bt[i, blk] = cache.block_table(rids[i], g)[blk]
                    sm[i] = bt[i, blk] * page
            window = cache.groups[g].window
            if window > 0:
                # the last step's advance gave back the pages that the window has passed: their
                # blocks are -1 in the requests' tables, and so they are here
                first_live = np.maximum(positions - window + 1, 0) // page
                released = np.arange(bt.shape[1], dtype=np.int64)[None, :] < first_live[:, None]
                if (released & (bt >= 0)).any():
                    bt = np.where(released, np.int32(-1), bt)
            tables.append(bt)
            slots.append(sm)
        return StepLayout(
            n_tokens=n, n_seqs=n, n_decode=n, row_of_entry=prev.row_of_entry, tokens=np.zeros(n, dtype=np.int32),
            positions=positions, token_seq=prev.token_seq, qo_indptr=prev.qo_indptr, kv_lens=positions + 1,
            slot_ids=prev.slot_ids, logit_rows=prev.logit_rows, block_tables=tables, slot_mappings=slots,
            page_sizes=list(cache.page_sizes), max_q_len=1, max_kv_len=int(positions.max()) + 1,
        )

    # ------------------------------------------------------------------ one step ahead
    def prepare_decode(self) -> Optional["PreparedDecode"]:
        """Call after a decode step, while the GPU is still busy with it: everything of the next
        decode step of the same requests (one token each, the same wanted places) that does not
        depend on the tokens is done now, the plan made, its pages taken, the upload buffer filled.
        ``step_prepared`` then only needs the tokens.  None when there is nothing to prepare: the
        last step was no decode step, pages are short, the step's shape has no recorded graph yet.  A preparation that is never used costs nothing but the pages it took
        early, which their requests keep, and would have taken with the step anyway."""
        if self.graphs is None or self._last_decode is None:
            return None
        rids, wants, prev, epoch = self._last_decode
        if epoch != self.cache.epoch:
            return None
        layout = self._next_decode_layout()
        if layout is None:
            return None
        graph = self.graphs.recorded(layout)
        if graph is None:
            return None  # the pages are taken all the same; the step finds them when it is planned
        graph.pack(layout)
        return PreparedDecode(rids, wants, prev, layout, graph, self.cache.epoch)

    @torch.inference_mode()
    def step_prepared(self, prepared: "PreparedDecode", entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """``step(entries)`` by way of what ``prepare_decode`` prepared.  Returns the logits, or
        None, with nothing run, when the entries are not the step that was prepared (other
        requests, more tokens, other wanted places) or the preparation is out of date (another step
        ran, requests came or went): ``step`` then does the whole work."""
        last = self._last_decode
        if last is None or last[2] is not prepared.previous or prepared.epoch != self.cache.epoch:
            return None
        if len(entries) != len(prepared.rids):
            return None
        tokens = prepared.layout.tokens
        for i, (e, rid, want) in enumerate(zip(entries, prepared.rids, prepared.wants)):
            if e.rid != rid or len(e.tokens) != 1 or list(e.want) != want:
                return None
            if not 0 <= e.tokens[0] < self.vocab_size:
                return None  # step() says what is wrong with it
            tokens[i] = e.tokens[0]
        prepared.graph.set_tokens(tokens)
        logits = prepared.graph.launch()
        for rid in prepared.rids:
            self.cache.advance(rid, 1)
        self._last_decode = (prepared.rids, prepared.wants, prepared.layout, self.cache.epoch)
        self.steps_run += 1
        self.tokens_run += len(prepared.rids)
        return logits

    @torch.inference_mode()
    def step_prepared_on_device(self, prepared: "PreparedDecode", rids: Sequence[Hashable], token_ids: torch.Tensor) -> Optional[torch.Tensor]:
        """``step_prepared`` for a step whose tokens the host does not know yet: ``token_ids`` is what
        the sampling kernel returned for the last step, still on the device, one token for each of
        ``rids``, which must be the prepared requests in their order, each wanting its one row.  The
        step is queued behind the sampling; nothing waits.  The caller vouches for the tokens (the
        sampling kernel returns token ids) and has to cope with a request that turns out to have
        ended with the token it is fed here: its row is then wasted, the other rows are as good
        as any.  None, with nothing run, when the preparation does not fit.  The logits returned are
        the recording's own: they hold until the engine's next step is queued, which is long enough
        for whoever queues the sampling first."""
        last = self._last_decode
        if last is None or last[2] is not prepared.previous or prepared.epoch != self.cache.epoch:
            return None
        if list(rids) != list(prepared.rids) or any(want != [0] for want in prepared.wants):
            return None
        if token_ids.dtype != torch.int32 or token_ids.numel() != len(prepared.rids) or token_ids.device != prepared.graph.dev.device:
            return None
        logits = prepared.graph.launch(token_ids, lend=True)
        for rid in prepared.rids:
            self.cache.advance(rid, 1)
        self._last_decode = (prepared.rids, prepared.wants, prepared.layout, self.cache.epoch)
        self.steps_run += 1
        self.tokens_run += len(prepared.rids)
        return logits

    def plan(self, entries: Sequence[StepEntry]) -> StepLayout:
        """Reserve pages for the step's tokens (all or nothing) and lay the step out."""
        # decode steps follow one another with the same requests: such a step is planned from the
        # last one's plan
        if self._last_decode is not None:
            last = self._last_decode
            layout = self._plan_next_decode(entries)
            self._last_decode = None
            if layout is not None:
                self._last_decode = (last[0], last[1], layout, self.cache.epoch)
                return layout
        layout = self._plan_general(entries)
        if layout.n_decode == layout.n_seqs:
            self._last_decode = (
                tuple(e.rid for e in entries), tuple(list(e.want) for e in entries), layout, self.cache.epoch
            )
        return layout

    def _plan_general(self, entries: Sequence[StepEntry]) -> StepLayout:
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise ValueError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if not self.cache.has(e.rid):
                raise KeyError(f"request {e.rid!r} is not live (admit it first)")
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.rid!r}: an entry needs at least one token")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= self.vocab_size:
                raise ValueError(
                    f"request {e.rid!r}: token id {lo if lo < 0 else hi} outside the vocabulary of {self.vocab_size}"
                )
            if self.cache.num_tokens(e.rid) + n > self.max_model_len:
                raise ValueError(
                    f"request {e.rid!r}: {self.cache.num_tokens(e.rid)} + {n} tokens exceed max_model_len={self.max_model_len}"
                )
        # all-or-nothing over the whole batch: count the pages the step takes from every pool
        need = [0] * len(self.cache.pools)
        for e in entries:
            for gi, pages in enumerate(self.cache.new_pages_needed(e.rid, len(e.tokens))):
                need[gi] += pages
        for gi, pool in enumerate(self.cache.pools):
            if need[gi] > pool.free_count:
                raise OutOfPages(
                    f"step needs {need[gi]} new pages in group {self.cache.groups[gi].name}, {pool.free_count} are free"
                )
        starts = [self.cache.extend(e.rid, len(e.tokens)) for e in entries]
        slots = [self.cache.slot(e.rid) for e in entries]
        tables = [[self.cache.block_table_array(e.rid, g) for e in entries] for g in range(len(self.cache.groups))]
        return build_step_layout(entries, starts, slots, tables, self.cache.page_sizes)

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one batch; returns float32 logits [number of wanted places, vocab], in the order
        of the entries and of their ``want`` lists."""
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        layout = self.plan(entries)
        try:
            if self.graphs is not None and layout.n_decode == layout.n_seqs:
                logits = self.graphs.run(layout)
            else:
                ctx = upload(layout, self.device)
                logits = self.model.forward(ctx, self.cache)
        except BaseException:
            # nothing of the step is booked: the pages taken for it go back, and no later step is
            # planned from this one's plan
            self._last_decode = None
            for e in entries:
                self.cache.truncate(e.rid, self.cache.num_tokens(e.rid))
            raise
        for e in entries:
            self.cache.advance(e.rid, len(e.tokens))
        self.steps_run += 1
        self.tokens_run += layout.n_tokens
        return logits
