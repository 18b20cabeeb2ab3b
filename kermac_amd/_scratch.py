"""Device memory that the operators use beside their operands and their result.

The reference's operators allocate nothing but ``out`` (README.md:69,135).  Here the default routes of
large calls do: a workspace about as large as the operands for the matrix-core and fixed-point routes,
partial sums for launches that are cut over the contraction, panels of the kernel matrix for the
coefficient product.  All of it goes through this module, which offers two controls:

``set_max_scratch_bytes(n)`` (or ``KERMAC_AMD_MAX_SCRATCH_BYTES=n`` for the process)
    the most one operator call may take, all buffers together; ``0`` is the reference's behaviour --
    nothing but ``out``: every call then runs the kernels that need no workspace (the one-step
    matrix-core kernels or the direct kernel, uncut launches, the fused coefficient kernel).
    ``None`` (the default) sets no limit.

``with kermac.scratch(buffer): ...``
    the calls the current host thread makes inside the block take their buffers from ``buffer`` (a
    1-D ``torch.uint8`` tensor on the operands' device) and allocate nothing at all; what does not
    fit is done without.  The buffer is handed out again from its start by every operator call, so
    calls that share it must be ordered on one stream, and its contents mean nothing between calls.

A route that is refused its memory falls back to the kernels that need none; results keep their
tolerance, and for a given shape and setting the choice is always the same.
"""
from __future__ import annotations

import contextlib
import functools
import os
import threading
from typing import Optional

import torch

_ALIGN = 256


def _parse_limit(text):
    if text is None or text == "":
        return None
    value = int(text)
    if value < 0:
        raise ValueError("KERMAC_AMD_MAX_SCRATCH_BYTES must not be negative")
    return value


_process = {"limit": _parse_limit(os.environ.get("KERMAC_AMD_MAX_SCRATCH_BYTES"))}
_thread = threading.local()


def set_max_scratch_bytes(limit: Optional[int]) -> None:
    """The most device memory one operator call may allocate beside ``out`` (bytes, all of its buffers
    together); 0: nothing, None: no limit."""
    if limit is not None and limit < 0:
        raise ValueError("the limit must not be negative")
    _process["limit"] = None if limit is None else int(limit)


def get_max_scratch_bytes() -> Optional[int]:
    return _process["limit"]


def _state():
    state = getattr(_thread, "state", None)
    if state is None:
        state = _thread.state = {"buffers": [], "depth": 0, "used": 0}
    return state


@contextlib.contextmanager
def scratch(buffer: torch.Tensor):
    """Operator calls of this host thread inside the block take their buffers from ``buffer`` and allocate nothing."""
    if not isinstance(buffer, torch.Tensor) or buffer.dtype != torch.uint8 or buffer.dim() != 1 or not buffer.is_contiguous():
        raise TypeError("scratch(buffer): a contiguous 1-D torch.uint8 tensor is needed")
    state = _state()
    state["buffers"].append(buffer)
    try:
        yield buffer
    finally:
        state["buffers"].pop()


@contextlib.contextmanager
def operator_call():
    """Wraps one public operator call: the limit and a supplied buffer are counted per outermost call
    (an operator that calls another one shares its budget)."""
    state = _state()
    if state["depth"] == 0:
        state["used"] = 0
    state["depth"] += 1
    try:
        yield
    finally:
        state["depth"] -= 1


def operator(function):
    """Decorator of the public operators: the body runs inside ``operator_call()``; signature and docstring stay."""
    @functools.wraps(function)
    def wrapped(*args, **kwargs):
        with operator_call():
            return function(*args, **kwargs)
    return wrapped


def allocate(nbytes: int, device: torch.device) -> Optional[torch.Tensor]:
    """``nbytes`` of device memory as a 256-byte aligned 1-D uint8 tensor, or None when the limit, the supplied
    buffer or the device's free memory does not allow it."""
    nbytes = int(nbytes)
    state = _state()
    if state["buffers"]:
        buffer = state["buffers"][-1]
        if buffer.device != device:
            return None
        start = -(-(buffer.data_ptr() + state["used"]) // _ALIGN) * _ALIGN - buffer.data_ptr()
        if start + nbytes > buffer.numel():
            return None
        state["used"] = start + nbytes
        return buffer[start:start + nbytes]
    limit = _process["limit"]
    if limit is not None and state["used"] + nbytes > limit:
        return None
    try:
        taken = torch.empty(nbytes, dtype=torch.uint8, device=device)
    except torch.cuda.OutOfMemoryError:
        return None
    state["used"] += nbytes
    return taken


def allocate_floats(shape, device: torch.device) -> Optional[torch.Tensor]:
    """A contiguous fp32 tensor of ``shape`` from ``allocate``."""
    count = 1
    for extent in shape:
        count *= int(extent)
    taken = allocate(4 * count, device)
    return None if taken is None else taken.view(torch.float32).view(*shape)
