"""Decode steps recorded as HIP graphs.

A decode step launches a few hundred small kernels; issued one by one from Python they take
longer to launch than to run.  A step whose every request brings exactly one token has a fixed
shape, so its launches are recorded once into a HIP graph and replayed: the step's plan is copied
into buffers at fixed addresses, the graph runs, and the logits appear in a fixed tensor.  (The
reference reaches for ``torch.compile(mode="reduce-overhead")`` here:
torchllms/inference/llm.py:202-283.)

A graph is keyed by what fixes its launches: the number of requests, the number of wanted logit
rows, a cap on the context length (a power of two or one and a half times one), which bounds the
block tables' width and fixes the key splits of the decode attention, and whether the requests
differ much in length, which makes those splits shorter.  No memset node is recorded: buffers are written by
kernels only.
"""

from __future__ import annotations

import gc
from typing import Dict, Tuple

import torch

from .context import make_context, pack_into, section_offsets, section_shapes
from .layout import StepLayout

MIN_CONTEXT_CAP = 512


def context_cap(max_kv_len: int) -> int:
    """The smallest of 512, 768, 1,024, 1,536, 2,048, ... that holds ``max_kv_len``.  The decode
    attention cuts the keys into splits for the cap, not for the contexts of the day, so a cap far
    above them gives splits that are too long and too few: with powers of two alone, 8 requests of
    2,176 tokens got the splits of 4,096 and the kernel took 24.9 us instead of 21.9."""
    cap = MIN_CONTEXT_CAP
    while cap < max_kv_len:
        if cap // 2 * 3 >= max_kv_len:
            return cap // 2 * 3
        cap *= 2
    return cap


class DecodeGraph:
    """One recorded decode step.  It refers to the model and the cache, never to the engine that
    owns it: a reference cycle would leave the graph to the cyclic garbage collector, which may
    run, and destroy the graph, in the middle of somebody else's stream capture."""

    def __init__(self, model, cache, device, layout: StepLayout, cap: int, pool=None, uneven: bool = False):
        self.model = model
        self.cache = cache
        self.cap = cap
        self.uneven = uneven
        self.pool = pool
        widths = [-(-cap // page) for page in layout.page_sizes]  # a group's block table up to the context cap
        self.shapes = section_shapes(layout.n_tokens, layout.n_seqs, layout.logit_rows.size, widths)
        self.offsets, total = section_offsets(self.shapes)
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=device)
        self.copied = torch.cuda.Event()
        self.graph = None
        self.logits = None
        self.replays = 0

    def pack(self, layout: StepLayout) -> None:
        """The plan into the pinned buffer.  May run while an earlier replay is still busy on the
        GPU: that replay reads the device buffer, which only ``_upload`` touches."""
        if self.replays or self.graph is not None:
            self.copied.synchronize()  # the pinned buffer is free again
        pack_into(self.host_np, layout, self.shapes, self.offsets)

    def set_tokens(self, tokens) -> None:
        """The token ids of an already packed plan (they are the first section of the buffer)."""
        off = self.offsets[0]
        self.host_np[off : off + len(tokens)] = tokens

    def token_section(self, n: int) -> torch.Tensor:
        """Where the recording reads the step's first ``n`` token ids: whoever produces them on the
        device may write them there and hand this tensor to ``launch``."""
        off = self.offsets[0]
        return self.dev[off : off + n]

    def _upload(self, but_tokens: int = 0) -> None:
        """The packed plan to the device; without its first ``but_tokens`` token ids if they are there already."""
        start = self.offsets[0] + but_tokens if but_tokens else 0
        assert self.offsets[0] == 0  # the token ids lead the buffer
        self.dev[start:].copy_(self.host[start:], non_blocking=True)
        self.copied.record()

    def _load(self, layout: StepLayout) -> None:
        self.pack(layout)
        self._upload()

    @torch.inference_mode()
    def first_run(self, layout: StepLayout) -> torch.Tensor:
        """Run the step eagerly (this is the step's real execution), then record the same launches.
        In inference mode whoever calls: so is every other capture of this package (see
        ``ops.tune_linear`` for why they must agree)."""
        self._load(layout)
        ctx = make_context(layout, self.dev, self.shapes, self.offsets, decode_longest=self.cap, decode_uneven=self.uneven)
        logits = self.model.forward(ctx, self.cache)
        result = logits.clone()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        # what the eager run derived from the step's plan (tables of cosines, ...) belongs to that
        # run: the recording has to contain the kernels that derive it anew from the fixed buffers
        ctx.scratch.clear()
        # nothing may be destroyed while the stream is capturing (a graph of an engine that is
        # garbage, say): the collector stays off until the capture has ended
        gc_was_on = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=self.pool):
                self.logits = self.model.forward(ctx, self.cache)
        finally:
            if gc_was_on:
                gc.enable()
        self.graph = graph
        self.ctx = ctx
        return result

    def replay(self, layout: StepLayout) -> torch.Tensor:
        self.pack(layout)
        return self.launch()

    def launch(self, tokens_on_device: torch.Tensor = None, lend: bool = False) -> torch.Tensor:
        """Upload the packed plan and replay.  ``tokens_on_device``: the step's token ids as an int32
        tensor on the device, which take the place of the plan's (they need not be known on the host:
        the copy is queued behind whatever produces them; none is needed when they were written into
        ``token_section`` itself).  ``lend``: return the recording's own logits,
        which the next replay overwrites, instead of a copy (a copy of 33 MB at 64 rows, and one more
        small launch between two steps at any size)."""
        if tokens_on_device is None:
            self._upload()
        else:
            n = tokens_on_device.numel()
            section = self.token_section(n)
            if tokens_on_device.data_ptr() == section.data_ptr():  # written in place: nothing to copy
                self._upload(but_tokens=n)
            else:
                self._upload()
                section.copy_(tokens_on_device)
        self.graph.replay()
        self.replays += 1
        return self.logits if lend else self.logits.clone()


class DecodeGraphs:
    """The engine's recorded decode steps, by (requests, wanted rows, context cap, uneven lengths).

    Recording costs many times a step, so a shape is recorded only when it comes back: the first
    ``record_after`` steps of a shape run eagerly (while requests join one by one every step has a
    new shape that never returns).  All recordings share one memory pool: they are replayed one at
    a time and a step's logits are copied out before the next replay."""

    def __init__(self, model, cache, device, max_graphs: int = 128, record_after: int = 2):
        self.model = model
        self.cache = cache
        self.device = device
        self.max_graphs = max_graphs
        self.record_after = record_after
        self.graphs: Dict[Tuple[int, int, int, bool], DecodeGraph] = {}
        self.seen: Dict[Tuple[int, int, int, bool], int] = {}
        self.pool = None

    def key_of(self, layout: StepLayout) -> Tuple[int, int, int, bool]:
        return (layout.n_seqs, int(layout.logit_rows.size), context_cap(layout.max_kv_len), layout.decode_uneven)

    def recorded(self, layout: StepLayout):
        """The recording that would replay this plan, or None."""
        g = self.graphs.get(self.key_of(layout))
        return g if g is not None and g.graph is not None else None

    def run(self, layout: StepLayout) -> torch.Tensor:
        key = self.key_of(layout)
        cap, uneven = key[2], key[3]
        g = self.graphs.get(key)
        if g is not None:
            return g.replay(layout)
        count = self.seen.get(key, 0) + 1
        self.seen[key] = count
        if count <= self.record_after:
            from .context import upload

            return self.model.forward(upload(layout, self.device), self.cache)
        if len(self.graphs) >= self.max_graphs:
            self.graphs.pop(next(iter(self.graphs)))
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        g = DecodeGraph(self.model, self.cache, self.device, layout, cap, self.pool, uneven)
        logits = g.first_run(layout)
        # kept only once it holds a recording: a step that raised leaves nothing behind that a later
        # step of the same shape would try to replay
        self.graphs[key] = g
        return logits
