"""Device-side view of one step's plan, handed to every part."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List

import numpy as np
import torch

from .layout import StepLayout

_ALIGN = 4  # int32 entries: every section starts on a 16-byte boundary


@dataclass
class StepContext:
    """int32 device tensors of the step (see ``StepLayout`` for their meaning) and the host plan."""

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

    @property
    def n_tokens(self) -> int:
        return self.host.n_tokens

    @property
    def n_seqs(self) -> int:
        return self.host.n_seqs


def upload(layout: StepLayout, device) -> StepContext:
    """Pack all vectors of the plan into one buffer and copy it to the device once."""
    sections = [
        layout.tokens, layout.positions, layout.token_seq, layout.qo_indptr, layout.kv_lens,
        layout.slot_ids, layout.logit_rows,
    ]
    for bt, sm in zip(layout.block_tables, layout.slot_mappings):
        sections.append(bt.reshape(-1))
        sections.append(sm)
    offsets = []
    total = 0
    for s in sections:
        offsets.append(total)
        total += -(-s.size // _ALIGN) * _ALIGN
    buf = np.zeros(max(total, _ALIGN), dtype=np.int32)
    for off, s in zip(offsets, sections):
        buf[off : off + s.size] = s
    dev = torch.from_numpy(buf).to(device)
    views = [dev[off : off + s.size] for off, s in zip(offsets, sections)]
    bts, sms = [], []
    for g, bt in enumerate(layout.block_tables):
        bts.append(views[7 + 2 * g].view(bt.shape))
        sms.append(views[8 + 2 * g])
    return StepContext(
        host=layout,
        tokens=views[0],
        positions=views[1],
        token_seq=views[2],
        qo_indptr=views[3],
        kv_lens=views[4],
        slot_ids=views[5],
        logit_rows=views[6],
        block_tables=bts,
        slot_mappings=sms,
    )
