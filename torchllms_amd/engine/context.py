"""Device-side view of one step's plan, handed to every part."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from .layout import StepLayout

_ALIGN = 4  # int32 entries: every section starts on a 16-byte boundary


@dataclass
class StepContext:
    """int32 device tensors of the step (see ``StepLayout`` for their meaning) and the host plan.

    ``decode_longest``: when set, an upper bound of the key range any single-token row sees; kernels
    then size their launches from it instead of from the host plan (a step recorded in a HIP graph
    must not depend on values that change from replay to replay).  ``decode_uneven`` likewise fixes
    what the host plan's property of that name would say.
    """

    host: StepLayout
    tokens: torch.Tensor
    positions: torch.Tensor
    token_seq: torch.Tensor
    qo_indptr: torch.Tensor
    kv_lens: torch.Tensor
    slot_ids: torch.Tensor
    logit_rows: torch.Tensor
    block_tables: List[torch.Tensor] = field(default_factory=list)
    slot_mappings: List[torch.Tensor] = field(default_factory=list)
    decode_longest: Optional[int] = None
    decode_uneven: Optional[bool] = None
    #: what kernels derive from the plan once per step and share between layers
    scratch: dict = field(default_factory=dict)

    @property
    def n_tokens(self) -> int:
        return self.host.n_tokens

    @property
    def n_seqs(self) -> int:
        return self.host.n_seqs


def section_shapes(n_tokens: int, n_seqs: int, n_out: int, table_widths: Sequence[int]) -> List[Tuple[int, ...]]:
    """Shapes of the packed sections, in order: tokens, positions, token_seq, qo_indptr, kv_lens,
    slot_ids, logit_rows, then per group its block table and its slot mapping."""
    shapes: List[Tuple[int, ...]] = [(n_tokens,), (n_tokens,), (n_tokens,), (n_seqs + 1,), (n_seqs,), (n_seqs,), (n_out,)]
    for width in table_widths:
        shapes.append((n_seqs, width))
        shapes.append((n_tokens,))
    return shapes


def section_offsets(shapes: Sequence[Tuple[int, ...]]) -> Tuple[List[int], int]:
    offsets, total = [], 0
    for shape in shapes:
        offsets.append(total)
        total += -(-int(np.prod(shape)) // _ALIGN) * _ALIGN
    return offsets, max(total, _ALIGN)


def pack_into(buf: np.ndarray, layout: StepLayout, shapes, offsets) -> None:
    """Write the plan's vectors into ``buf`` at ``offsets``; block tables are padded with -1 to the
    widths that ``shapes`` give."""
    sections = [layout.tokens, layout.positions, layout.token_seq, layout.qo_indptr, layout.kv_lens, layout.slot_ids, layout.logit_rows]
    for s, shape, off in zip(sections, shapes, offsets):
        if s.shape != shape:
            raise ValueError(f"step plan does not fit the buffer: section of shape {s.shape}, room for {shape}")
        buf[off : off + s.size] = s
    for g, (bt, sm) in enumerate(zip(layout.block_tables, layout.slot_mappings)):
        shape, off = shapes[7 + 2 * g], offsets[7 + 2 * g]
        if bt.shape[0] != shape[0] or bt.shape[1] > shape[1]:
            raise ValueError(f"block table of shape {bt.shape} does not fit {shape}")
        view = buf[off : off + shape[0] * shape[1]].reshape(shape)
        view[:, : bt.shape[1]] = bt
        view[:, bt.shape[1] :] = -1
        off = offsets[8 + 2 * g]
        buf[off : off + sm.size] = sm


def make_context(layout: StepLayout, dev: torch.Tensor, shapes, offsets, decode_longest: Optional[int] = None,
                 decode_uneven: Optional[bool] = None) -> StepContext:
    views = [dev[off : off + int(np.prod(shape))].view(shape) for shape, off in zip(shapes, offsets)]
    n_groups = (len(shapes) - 7) // 2
    return StepContext(
        host=layout,
        tokens=views[0],
        positions=views[1],
        token_seq=views[2],
        qo_indptr=views[3],
        kv_lens=views[4],
        slot_ids=views[5],
        logit_rows=views[6],
        block_tables=[views[7 + 2 * g] for g in range(n_groups)],
        slot_mappings=[views[8 + 2 * g] for g in range(n_groups)],
        decode_longest=decode_longest,
        decode_uneven=decode_uneven,
    )


def upload(layout: StepLayout, device) -> StepContext:
    """Pack all vectors of the plan into one buffer and copy it to the device once."""
    shapes = section_shapes(layout.n_tokens, layout.n_seqs, layout.logit_rows.size, [bt.shape[1] for bt in layout.block_tables])
    offsets, total = section_offsets(shapes)
    buf = np.zeros(total, dtype=np.int32)
    pack_into(buf, layout, shapes, offsets)
    return make_context(layout, torch.from_numpy(buf).to(device), shapes, offsets)
