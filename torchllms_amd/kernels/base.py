"""What the kernel wrappers share: dtype codes, argument checks, and a matrix product that is still
split along K (the norm that adds it up and the product kernels that leave it both need the type)."""

from __future__ import annotations

from typing import Optional

import torch

from .lib import KernelError, check, core, device_facts, variant  # noqa: F401

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {dtype}; kernels take float32 and bfloat16") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors (there is no CPU path)")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _i32(t: Optional[torch.Tensor], what: str) -> None:
    if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous int32 tensor")


class Unfinished:
    """A result whose last kernel has not run yet, because the kernel that reads it can do that work
    on the way.  ``resolve()`` runs it and returns the tensor; ``resolved(x)`` does so for anything."""

    def resolve(self) -> torch.Tensor:
        raise NotImplementedError


class SplitSums(Unfinished):
    """A matrix product that was split along K and not yet added up: ``partial`` float32
    [splits, rows, columns].  The product is the sum of the slices in their order, rounded to
    ``dtype``; ``rmsnorm`` takes it as ``delta`` and adds the slices while it reads them, which
    saves the kernel that would otherwise do nothing else."""

    def __init__(self, partial: torch.Tensor, dtype: torch.dtype):
        self.partial = partial
        self.dtype = dtype

    @property
    def shape(self):
        return tuple(self.partial.shape[1:])

    def resolve(self) -> torch.Tensor:
        splits, m, n = self.partial.shape
        out = torch.empty((m, n), dtype=self.dtype, device=self.partial.device)
        check(core().tl_gemm_wide_reduce(self.partial.data_ptr(), out.data_ptr(), out.stride(0), m, n, splits, dtype_code(self.dtype), _stream()))
        return out


def resolved(x):
    """``x`` as a tensor: an ``Unfinished`` result (a ``SplitSums``, a ``PendingProduct``, ``NormedRows``)
    is finished, a tensor is returned as it is.  For code that does arithmetic of its own on what a
    norm, mixer or feed-forward returned."""
    return x.resolve() if isinstance(x, Unfinished) else x
