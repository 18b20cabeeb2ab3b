"""Layout analysis and small helpers shared by the operators.

Mirrors the public helper names of the reference's ``src/kermac/common.py`` so
that code written against it keeps working: ``Majorness``, ``Alignment``,
``FillMode``, ``TensorStats`` / ``tensor_stats``, ``merge_batch_size``,
``ceil_div``, ``CudaTimer`` and ``PyTorchStreamWrapper``.
"""
from __future__ import annotations

import os
from enum import Enum, auto
from typing import Optional, Tuple, Union

import torch


class Majorness(Enum):
    """Which of the last two dimensions is contiguous (reference: common.py:5-7)."""
    COL_MAJOR = auto()   # stride(-2) == 1: the row index is the fast one
    ROW_MAJOR = auto()   # stride(-1) == 1: torch's default


class Alignment(Enum):
    """Whether 16-byte (4 x fp32) accesses are legal (reference: common.py:10-12)."""
    ALIGN_1 = auto()
    ALIGN_4 = auto()


class FillMode(Enum):
    UPPER = auto()
    LOWER = auto()


class PyTorchStreamWrapper:
    """Adapter exposing a torch stream through the ``__cuda_stream__`` protocol
    (reference: common.py:18-24).  On ROCm the handle is a ``hipStream_t``."""

    def __init__(self, pt_stream):
        self.pt_stream = pt_stream

    def __cuda_stream__(self):
        return (0, self.pt_stream.cuda_stream)

    @property
    def handle(self) -> int:
        return int(self.pt_stream.cuda_stream)


class CudaTimer:
    """Event timer on the current stream; ``stop()`` returns milliseconds
    (reference: common.py:26-42).  torch keeps the ``cuda`` names on ROCm."""

    def __init__(self):
        if not torch.cuda.is_available():
            raise RuntimeError("CUDA is not available")
        self.start_event = torch.cuda.Event(enable_timing=True)
        self.end_event = torch.cuda.Event(enable_timing=True)

    def start(self):
        self.start_event.record()

    def stop(self):
        self.end_event.record()
        self.end_event.synchronize()
        return self.start_event.elapsed_time(self.end_event)


def launch_cuts_enabled() -> bool:
    """The Python layer cuts launches that would leave CUs idle into one batched launch over
    ranges of the contracted index plus a sum of partial results, which needs a temporary
    buffer (up to 512 MB).  KERMAC_AMD_NO_CUT=1 launches every call exactly as it was given."""
    return os.environ.get("KERMAC_AMD_NO_CUT", "0") in ("", "0")


def ceil_div(x, d):
    return int(-(-x // d))


def merge_batch_size(
    name: str,
    L,
    a: Union[float, torch.Tensor, None],
    expected_dims: int,
    can_be_none: bool = False,
):
    """Fold operand ``a`` into the running batch count ``L``.

    An operand with exactly ``expected_dims`` dimensions is unbatched; one extra
    leading dimension is its batch, which must be 1 or agree with every other
    non-1 batch (reference: common.py:47-70).
    """
    if a is None:
        if can_be_none:
            return L
        raise ValueError(f"{name} is none, but can_be_none is False")
    if isinstance(a, float):
        if expected_dims == 0:
            return L
        raise ValueError(f"{name} is a float but expected_dims is {expected_dims}")
    if isinstance(a, torch.Tensor):
        extra = a.dim() - expected_dims
        if extra == 0:
            return L
        if extra == 1:
            own = a.size(0)
            if own != 1 and L != 1 and own != L:
                raise ValueError(f"{name} batch size of {own} does not match with another non-one batch size, {L}")
            return max(L, own)
        raise ValueError(
            f"{name} does have the right number of dimensions, expected_dims is "
            f"{expected_dims} or {expected_dims + 1}, got {a.dim()}"
        )
    # The reference falls through and returns None here; failing early is kinder.
    raise TypeError(f"{name} must be a float or a torch.Tensor, got {type(a).__name__}")


class TensorStats:
    """Batch count/stride, majorness, alignment and leading dimension of a 2-D or
    batched 3-D fp32 tensor (reference: common.py:72-141).

    * a 2-D tensor, or a 3-D one whose batch dimension is 1, broadcasts over the
      batch (batch stride 0);
    * ``ROW_MAJOR`` needs ``stride(-1) == 1`` and ``stride(-2) >= cols``;
      ``COL_MAJOR`` needs ``stride(-2) == 1`` and ``stride(-1) >= rows``; anything
      else is rejected;
    * ``ALIGN_4`` is only ever reported for ``COL_MAJOR`` tensors, as in the
      reference; the launch layer separately checks whether 128-bit accesses
      are legal for row-major operands.
    """

    __slots__ = ("_shape", "_num_batches", "_batch_stride", "_majorness", "_alignment", "_ld")

    def __init__(self, tensor: torch.Tensor):
        if tensor.dim() not in (2, 3):
            raise ValueError("Input tensor must be 2 or 3-dimensional")
        if tensor.dtype != torch.float32:
            raise TypeError("Input tensor must have dtype torch.float32")

        batched = tensor.dim() == 3
        self._num_batches = tensor.size(0) if batched else 1
        self._batch_stride = tensor.stride(0) if batched and self._num_batches != 1 else 0

        rows, cols = tensor.size(-2), tensor.size(-1)
        row_stride, col_stride = tensor.stride(-2), tensor.stride(-1)
        self._shape = (self._num_batches, rows, cols)

        if col_stride == 1 and row_stride >= cols:
            self._majorness = Majorness.ROW_MAJOR
        elif row_stride == 1 and col_stride >= rows:
            self._majorness = Majorness.COL_MAJOR
        else:
            raise ValueError(
                f"Tensor has non-standard memory layout: strides={tensor.stride()}, shape={tensor.size()}"
            )

        self._ld = max(row_stride, col_stride)
        sixteen_byte = tensor.data_ptr() % 16 == 0 and self._ld % 4 == 0
        if self._majorness is Majorness.COL_MAJOR and sixteen_byte:
            self._alignment = Alignment.ALIGN_4
        else:
            self._alignment = Alignment.ALIGN_1

    @property
    def shape(self) -> Tuple[int, int, int]:
        return self._shape

    @property
    def majorness(self) -> Majorness:
        return self._majorness

    @property
    def alignment(self) -> Alignment:
        return self._alignment

    @property
    def num_batches(self) -> int:
        return self._num_batches

    @property
    def batch_stride(self) -> int:
        return self._batch_stride

    @property
    def leading_dimension_stride(self) -> int:
        return self._ld


def tensor_stats(tensor: torch.Tensor) -> TensorStats:
    return TensorStats(tensor)
