"""Context-local options of the device path.

Three settings steer how the HIP library is driven: how rows whose label is
``ignore_index`` are compacted away, how many bytes the staging panel between
the contractions may take, and whether the gradients are formed during the
forward (three contractions) or by a backward that recomputes the logits
(four).  All are ``contextvars``: a value
set with the context managers below (or passed per call where a function takes
the keyword) is seen by the calling thread / task only, so two trainers in one
process can choose differently.  The reference's extension has no such
settings; its block size comes from ``native_ce_block_size``
(dllm_parallel/core/kernels/runtime.py) per call in the same spirit.
"""

from __future__ import annotations

import contextlib
import contextvars

# How the device path deals with rows whose label is ``ignore_index``:
#   "sync"   (default) compact them away on the device and read the count of
#            loss-bearing rows back once, so every launch is sized exactly (the
#            one host synchronisation the reference's call sites incur as well,
#            nemotron/model.py:4244-4248);
#   "device" compact them away without any host read-back: launches are sized
#            for all rows and the kernels take the count from device memory, so
#            the whole loss (forward and backward) can be recorded into a HIP
#            graph;
#   "none"   no compaction: the caller has compacted already (the reference's
#            call sites do) or accepts GEMM work on ignored rows; the kernels
#            zero their loss and gradient like the reference operator.
COMPACTION_MODES = ("sync", "device", "none")

_compaction = contextvars.ContextVar("tlce_compaction_mode", default="sync")
# 0 selects the library default: 2.5 GiB for the panel of exponentiated logits of the
# forward that leaves the gradients, 1 GiB for the recomputing backward's panel of logit
# gradients
_panel_bytes = contextvars.ContextVar("tlce_panel_bytes", default=0)


# When the gradients are formed:
#   "forward"   (default) during the forward, while the logits of a block of rows
#               exist: 3 contractions per step instead of 4.  Taken where the
#               library supports it (bf16 inputs, no bias, head stored [V, H], H
#               and V multiples of 64) and a gradient is required; other calls
#               fall back to "recompute".  The forward then holds the float32
#               grad_hidden [M, H] and either the float32 grad_weight [V, H] or,
#               when all rows fit one block, its workspace, until the backward
#               scales and rounds them.  Per-token losses (reduction "none")
#               take this path with a frozen head, and with a trainable head
#               when all rows fit one block: grad_weight needs the per-row
#               upstream gradients inside its contraction, which then runs in
#               the backward;
#   "recompute" by a backward that recomputes the logits in vocabulary panels, as
#               the reference's backward does block by block
#               (fused_linear_ce_cuda.cu:618-791).
GRADIENT_MODES = ("forward", "recompute")
_gradients = contextvars.ContextVar("tlce_gradient_mode", default="forward")


def get_gradient_mode() -> str:
    return _gradients.get()


def _checked_gradient_mode(mode: str) -> str:
    if mode not in GRADIENT_MODES:
        raise ValueError(f"gradient mode must be one of {GRADIENT_MODES}")
    return mode


def set_gradient_mode(mode: str) -> str:
    """Sets the mode for the current context (thread / task); returns the old one."""
    old = _gradients.get()
    _gradients.set(_checked_gradient_mode(mode))
    return old


@contextlib.contextmanager
def gradient_mode(mode: str):
    token = _gradients.set(_checked_gradient_mode(mode))
    try:
        yield
    finally:
        _gradients.reset(token)


def _checked_mode(mode: str) -> str:
    if mode not in COMPACTION_MODES:
        raise ValueError(f"compaction mode must be one of {COMPACTION_MODES}")
    return mode


def get_compaction_mode() -> str:
    return _compaction.get()


def set_compaction_mode(mode: str) -> str:
    """Sets the mode for the current context (thread / task); returns the old one."""
    old = _compaction.get()
    _compaction.set(_checked_mode(mode))
    return old


@contextlib.contextmanager
def compaction_mode(mode: str):
    token = _compaction.set(_checked_mode(mode))
    try:
        yield
    finally:
        _compaction.reset(token)


def resolve_compaction(compaction: str | None) -> str:
    """A per-call choice if given, else the context's mode."""
    return _compaction.get() if compaction is None else _checked_mode(compaction)


def get_panel_bytes() -> int:
    return _panel_bytes.get()


def set_panel_bytes(nbytes: int) -> int:
    """Sets the panel budget for the current context (thread / task); returns the old one."""
    if nbytes < 0:
        raise ValueError("panel budget must be >= 0 bytes")
    old = _panel_bytes.get()
    _panel_bytes.set(int(nbytes))
    return old


@contextlib.contextmanager
def panel_budget(nbytes: int):
    """Bounds the staging panel between the contractions inside the block
    (0 = library default)."""
    if nbytes < 0:
        raise ValueError("panel budget must be >= 0 bytes")
    token = _panel_bytes.set(int(nbytes))
    try:
        yield
    finally:
        _panel_bytes.reset(token)
