"""Python entry points of the gfx950 fused LM-head cross-entropy library.

Same role and call signatures as the reference's binding shim
(dllm_parallel/core/kernels/chunked_linear_ce_native.py:61-182): ``forward``,
``backward`` and ``backward_frozen_weight`` take flattened tensors and return
``(losses, lse, valid_count)`` / ``(grad_hidden, grad_weight, grad_bias)``.
Added on top: the device compaction entry points (``compact_rows``,
``gather_rows``, ``scatter_rows``) and the optional ``row_idx`` / ``n_out``
arguments that let the kernels read compacted rows and write their results
straight into the un-compacted token axis.

torch is used here only to allocate outputs and workspaces on the caller's
device and to hand over the current stream; all arithmetic runs in the HIP
library through its C ABI.  There is no fallback: a missing library raises.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import _lib

_DTYPE_CODES = {
    torch.float32: _lib.DTYPE_F32,
    torch.float16: _lib.DTYPE_F16,
    torch.bfloat16: _lib.DTYPE_BF16,
}

from .options import get_panel_bytes, panel_budget  # noqa: F401  (panel_budget re-exported)


def _reduction_code(reduction: str) -> int:
    # same numbering as chunked_linear_ce_native.py:366-373 of the reference
    if reduction == "none":
        return _lib.REDUCTION_NONE
    if reduction == "sum":
        return _lib.REDUCTION_SUM
    if reduction == "mean":
        return _lib.REDUCTION_MEAN
    raise ValueError(f"unsupported reduction: {reduction}")


def _dtype_code(tensor: torch.Tensor) -> int:
    try:
        return _DTYPE_CODES[tensor.dtype]
    except KeyError as exc:
        raise RuntimeError(
            "native linear CE supports float32, float16, and bfloat16"
        ) from exc


def _ptr(tensor: Optional[torch.Tensor]) -> Optional[int]:
    if tensor is None or tensor.numel() == 0:
        return None
    return tensor.data_ptr()


def _dense(tensor: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned: the MFMA kernels load 16 bytes at a time.
    A contiguous view at an odd offset (``hidden[1:]`` with a row length that is
    not a multiple of 16 bytes) is copied; everything else passes through."""
    tensor = tensor.contiguous()
    if tensor.numel() and tensor.data_ptr() % 16:
        tensor = tensor.clone()
    return tensor


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    device = None
    for tensor in tensors:
        if tensor is None:
            continue
        if not tensor.is_cuda:
            raise RuntimeError("native linear CE expects device (HIP) tensors")
        if device is None:
            device = tensor.device
        elif tensor.device != device:
            raise RuntimeError("native linear CE expects all tensors on one device")
    assert device is not None
    return device


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    # torch's caching allocator hands out 512-byte aligned blocks
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def verify_device(device: torch.device | int | None = None) -> None:
    """Raises unless the device is a gfx950 GPU the library has code for."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index
    _lib.check(_lib.library().tlce_check_device(int(index or 0)), "tlce_check_device")


_DFLASH_LOSS_KINDS = frozenset({
    "paper_ce", "speculators_kl", "dflash", "dpace",
    "dpace-cumulative-confidence-only", "dpace-continuation-value-only",
})
# entry points each family of DFlash losses calls in the library
_DFLASH_SYMBOLS = {
    "paper_ce": ("tlce_forward", "tlce_backward", "tlce_compact_mask"),
    "speculators_kl": ("tlce_kl_workspace_bytes", "tlce_kl_forward", "tlce_kl_backward",
                       "tlce_compact_mask"),
    "ce_topk": ("tlce_ce_topk_forward_workspace_bytes", "tlce_ce_topk_backward_workspace_bytes",
                "tlce_ce_topk_forward", "tlce_ce_topk_backward", "tlce_compact_mask"),
}


def verify_dflash_symbols(*, loss_kind: str) -> None:
    """Start-up check of the DFlash executor: raises ``ValueError`` for an unknown
    loss kind and a loader error when the library is absent or lacks an entry
    point that loss needs, so that a missing build fails before the first step
    and not inside it (reference shim, chunked_linear_ce_native.py:353-363,
    which resolves its DFlash extension the same way)."""
    if loss_kind not in _DFLASH_LOSS_KINDS:
        raise ValueError(f"unsupported DFlash loss {loss_kind!r}")
    family = loss_kind if loss_kind in ("paper_ce", "speculators_kl") else "ce_topk"
    lib = _lib.library()          # raises NativeLibraryMissing when it has not been built
    for name in _DFLASH_SYMBOLS[family]:
        if not hasattr(lib, name):
            raise _lib.NativeLibraryMissing(
                f"{_lib.LIBRARY_PATH} does not export {name!r}, which DFlash loss "
                f"{loss_kind!r} needs; rebuild the library")


# ----------------------------------------------------------------- compaction --
def compact_rows(labels: torch.Tensor, ignore_index: int) -> tuple[torch.Tensor, int]:
    """``nonzero(labels != ignore_index).flatten()`` on the device.

    Returns the ascending int64 indices (a view of length ``count``) and the
    count.  Reading the count back is the one host synchronisation of the
    path, the same one the reference incurs at ``row_indices.numel()``
    (nemotron/model.py:4244-4248).
    """
    device = _require_device(labels)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    n = labels.numel()
    lib = _lib.library()
    with torch.cuda.device(device):
        row_idx = torch.empty(max(n, 1), dtype=torch.long, device=device)
        count = torch.empty(1, dtype=torch.long, device=device)
        ws = _workspace(lib.tlce_compact_workspace_bytes(n), device)
        _lib.check(
            lib.tlce_compact_rows(
                _ptr(labels), n, int(ignore_index), row_idx.data_ptr(), count.data_ptr(),
                ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_compact_rows",
        )
        m = int(count.item())
    return row_idx[:m], m


def compact_rows_device(labels: torch.Tensor, ignore_index: int) -> tuple[torch.Tensor, torch.Tensor]:
    """As ``compact_rows`` without the host read-back: returns the index buffer
    at full length ``n`` (only its first ``count`` entries are defined) and the
    count as a device int64 tensor of one element.  Nothing here synchronises,
    so the call can be recorded into a HIP graph."""
    device = _require_device(labels)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    n = labels.numel()
    lib = _lib.library()
    with torch.cuda.device(device):
        row_idx = torch.empty(max(n, 1), dtype=torch.long, device=device)
        count = torch.empty(1, dtype=torch.long, device=device)
        ws = _workspace(lib.tlce_compact_workspace_bytes(n), device)
        _lib.check(
            lib.tlce_compact_rows(
                _ptr(labels), n, int(ignore_index), row_idx.data_ptr(), count.data_ptr(),
                ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_compact_rows",
        )
    return row_idx[:n], count


def _mask_bytes(mask: torch.Tensor) -> torch.Tensor:
    mask = mask.reshape(-1)
    if mask.dtype == torch.bool:
        return mask.contiguous().view(torch.uint8)
    if mask.dtype == torch.uint8:
        return mask.contiguous()
    return (mask != 0).view(torch.uint8)


def compact_mask_device(mask: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``nonzero(mask).flatten()`` on the device without a host read-back: the
    index buffer at full length (its first ``count`` entries are defined) and the
    count as a device int64 tensor of one element.  ``mask`` is a bool / uint8
    tensor (anything else is compared with 0 first)."""
    device = _require_device(mask)
    flags = _mask_bytes(mask)
    n = flags.numel()
    lib = _lib.library()
    with torch.cuda.device(device):
        row_idx = torch.empty(max(n, 1), dtype=torch.long, device=device)
        count = torch.empty(1, dtype=torch.long, device=device)
        ws = _workspace(lib.tlce_compact_workspace_bytes(n), device)
        _lib.check(
            lib.tlce_compact_mask(
                _ptr(flags), n, row_idx.data_ptr(), count.data_ptr(),
                ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_compact_mask",
        )
    return row_idx[:n], count


def compact_mask(mask: torch.Tensor) -> tuple[torch.Tensor, int]:
    """``nonzero(mask).flatten()`` (ascending int64) and its length, read back
    once: the host synchronisation ``valid_indices.numel()`` costs the
    reference too (dflash/model.py:885)."""
    row_idx, count = compact_mask_device(mask)
    m = int(count.item())
    return row_idx[:m], m


def gather_loss_rows(
    hidden: torch.Tensor,
    labels: torch.Tensor,
    weights: torch.Tensor | None,
    row_idx: torch.Tensor,
    row_count: torch.Tensor,
    ignore_index: int,
    capacity: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
    """Hidden rows, labels and (optional) float32 loss weights of the first
    ``row_count`` positions in ``row_idx``, gathered in one launch with the
    count read on the device.  ``capacity`` bounds the count (default: all ``n``
    rows; a caller that has read the count back passes it).  The outputs have
    ``round_up(capacity, 64)`` rows; rows from the count up to the next
    multiple of 64 are zero / ignored / weight 0."""
    device = _require_device(hidden, labels, weights, row_idx, row_count)
    hidden = hidden.contiguous()
    labels = labels.reshape(-1).to(torch.long).contiguous()
    n, h = hidden.shape
    capacity = n if capacity is None else int(capacity)
    if labels.numel() != n or not 0 <= capacity <= n or row_idx.numel() < capacity:
        raise RuntimeError("gather_loss_rows: hidden, labels and row_idx lengths differ")
    if weights is not None:
        weights = weights.reshape(-1).to(torch.float32).contiguous()
        if weights.numel() != n:
            raise RuntimeError("gather_loss_rows: weights length differs")
    padded = (capacity + 63) // 64 * 64
    row_bytes = h * hidden.element_size()
    with torch.cuda.device(device):
        rows = torch.empty((padded, h), dtype=hidden.dtype, device=device)
        targets = torch.empty(padded, dtype=torch.long, device=device)
        w = None if weights is None else torch.empty(padded, dtype=torch.float32, device=device)
        if capacity:
            _lib.check(
                _lib.library().tlce_gather_loss_rows(
                    hidden.data_ptr(), labels.data_ptr(), _ptr(weights), row_idx.data_ptr(),
                    row_count.data_ptr(), capacity, padded, row_bytes, int(ignore_index),
                    rows.data_ptr(), targets.data_ptr(), _ptr(w), _stream(device),
                ),
                "tlce_gather_loss_rows",
            )
    return rows, targets, w


def compact_loss_rows(
    hidden: torch.Tensor,
    labels: torch.Tensor,
    weights: torch.Tensor | None,
    ignore_index: int,
    mode: str,
):
    """The row compaction in front of the loss kernels, by compaction mode.

    Returns ``(rows, targets, token_weights, row_idx, row_count, m)``: the
    operands the ``masked_loss_*`` / ``forward`` entry points take.  "none":
    the inputs as they are.  "sync": one scan, the count read back, then one
    fused gather of exactly the loss-bearing rows (padded with zero rows to a
    multiple of 64, which is what the count on the device, handed on as
    ``row_count``, licenses the kernels to read).  "device": the same without
    the read-back, every buffer sized for all rows."""
    n = hidden.shape[0]
    if mode == "none" or n == 0:
        return hidden, labels, weights, None, None, n
    row_idx, row_count = compact_rows_device(labels, ignore_index)
    if mode == "device":
        rows, targets, token_weights = gather_loss_rows(hidden, labels, weights, row_idx,
                                                        row_count, ignore_index)
        return rows, targets, token_weights, row_idx, row_count, n
    m = int(row_count.item())
    if m == n:
        return hidden, labels, weights, None, None, n
    if m == 0:
        return (hidden[:0], labels[:0], None if weights is None else weights[:0],
                row_idx[:0], None, 0)
    rows, targets, token_weights = gather_loss_rows(hidden, labels, weights, row_idx, row_count,
                                                    ignore_index, capacity=m)
    return rows, targets, token_weights, row_idx[:m], row_count, m


def segment_weighted_sum(
    values: torch.Tensor,
    weights: torch.Tensor | None,
    row_idx: torch.Tensor,
    segment_length: int,
    n_segments: int,
    row_count: torch.Tensor | None = None,
) -> torch.Tensor:
    """``out[s] = sum(values[r] * weights[r])`` over the compacted rows whose
    position ``row_idx[r]`` lies in sample ``s`` (positions ``[s * L, (s + 1) * L)``),
    float32 ``[n_segments]``, summed in a fixed order (no atomics): the
    reference's ``numerators.scatter_add_`` (dflash/model.py:925-937) for
    ascending ``row_idx``."""
    device = _require_device(values, weights, row_idx, row_count)
    values = values.reshape(-1).to(torch.float32).contiguous()
    m = values.numel()
    if weights is not None:
        weights = weights.reshape(-1).to(torch.float32).contiguous()
        if weights.numel() != m:
            raise RuntimeError("segment_weighted_sum: values and weights lengths differ")
    row_idx = row_idx.reshape(-1).to(torch.long).contiguous()
    if row_idx.numel() < m:
        raise RuntimeError("segment_weighted_sum: row_idx holds fewer entries than values")
    with torch.cuda.device(device):
        out = torch.empty(int(n_segments), dtype=torch.float32, device=device)
        _lib.check(
            _lib.library().tlce_segment_weighted_sum(
                _ptr(values), _ptr(weights), _ptr(row_idx), _ptr(row_count), m,
                int(segment_length), int(n_segments), _ptr(out), _stream(device),
            ),
            "tlce_segment_weighted_sum",
        )
    return out


def gather_rows(src: torch.Tensor, row_idx: torch.Tensor) -> torch.Tensor:
    """``src.index_select(0, row_idx)`` for a contiguous ``src`` (any trailing shape)."""
    device = _require_device(src, row_idx)
    src = src.contiguous()
    m = row_idx.numel()
    out = torch.empty((m, *src.shape[1:]), dtype=src.dtype, device=device)
    if m == 0 or src.numel() == 0:
        return out
    row_bytes = src.element_size() * (src.numel() // src.shape[0])
    with torch.cuda.device(device):
        _lib.check(
            _lib.library().tlce_gather_rows(
                src.data_ptr(), row_idx.data_ptr(), m, row_bytes, out.data_ptr(), _stream(device)
            ),
            "tlce_gather_rows",
        )
    return out


def scatter_rows(src: torch.Tensor, row_idx: torch.Tensor, n_rows: int) -> torch.Tensor:
    """Zero tensor of ``n_rows`` rows with ``out[row_idx[r]] = src[r]``."""
    device = _require_device(src, row_idx)
    src = src.contiguous()
    out = torch.empty((n_rows, *src.shape[1:]), dtype=src.dtype, device=device)
    lib = _lib.library()
    with torch.cuda.device(device):
        if out.numel():
            _lib.check(
                lib.tlce_fill_zero(out.data_ptr(), out.numel() * out.element_size(),
                                   _stream(device)),
                "tlce_fill_zero",
            )
        m = row_idx.numel()
        if m and src.numel():
            row_bytes = src.element_size() * (src.numel() // src.shape[0])
            _lib.check(
                lib.tlce_scatter_rows(
                    src.data_ptr(), row_idx.data_ptr(), m, row_bytes, out.data_ptr(),
                    _stream(device),
                ),
                "tlce_scatter_rows",
            )
    return out


# -------------------------------------------------------------------- forward --
def dim_first_in_place(weight: torch.Tensor, weight_dim_first: bool) -> bool:
    """True when a ``[H, V]`` head can be handed to the library as it is stored
    (``tlce_*_dim_first``: 16-bit dtypes, H and V multiples of 64)."""
    if not weight_dim_first or weight.dim() != 2 or weight.dtype not in _DTYPE_CODES:
        return False
    h, v = weight.shape
    return bool(_lib.library().tlce_dim_first_supported(int(h), int(v),
                                                        _DTYPE_CODES[weight.dtype]))


def _head_operand(weight: torch.Tensor, weight_dim_first: bool) -> tuple[torch.Tensor, bool]:
    """The head as the library takes it and whether that is the [H, V] form.  A
    [H, V] head is read in place where the kernels can (see
    ``dim_first_in_place``); otherwise it is re-laid to [V, H] once."""
    if dim_first_in_place(weight, weight_dim_first):
        return _dense(weight), True
    return (weight.t().contiguous() if weight_dim_first else _dense(weight)), False


def forward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    *,
    row_block_size: int,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
    compute_dtype: torch.dtype,
    weight_dim_first: bool,
    row_idx: torch.Tensor | None = None,
    n_out: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(losses [n_out] f32, lse [m] f32, valid_count [1] f32)``.

    ``row_block_size`` and ``compute_dtype`` are accepted for signature parity
    and ignored, as in the reference shim (chunked_linear_ce_native.py:61-94):
    tiling is fixed by the library's plan, arithmetic is in the input dtype
    with float32 accumulation.
    """
    del row_block_size, compute_dtype
    device = _require_device(hidden, weight, bias, labels, row_idx)
    if hidden.dim() != 2:
        raise RuntimeError("hidden must be flattened [N, D]")
    if weight.dim() != 2:
        raise RuntimeError("weight must be a matrix")
    if weight.dtype != hidden.dtype:
        raise RuntimeError("native linear CE expects hidden and weight of one dtype")
    hidden = _dense(hidden)
    weight, in_place = _head_operand(weight, weight_dim_first)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight.shape[1] if in_place else weight.shape[0]
    if weight.shape[0 if in_place else 1] != h or labels.numel() != m:
        raise RuntimeError("native linear CE shape mismatch")
    n_out = m if n_out is None else int(n_out)
    bias32 = None if bias is None else bias.to(torch.float32).contiguous()
    if bias32 is not None and bias32.numel() != v:
        raise RuntimeError("native linear CE bias shape mismatch")
    lib = _lib.library()
    code = _dtype_code(hidden)
    with torch.cuda.device(device):
        losses = torch.empty(n_out, dtype=torch.float32, device=device)
        lse = torch.empty(m, dtype=torch.float32, device=device)
        valid_count = torch.empty(1, dtype=torch.float32, device=device)
        ws = _workspace(lib.tlce_forward_workspace_bytes(m, h, v, code), device)
        entry = lib.tlce_forward_dim_first if in_place else lib.tlce_forward
        _lib.check(
            entry(
                _ptr(hidden), _ptr(weight), _ptr(bias32), _ptr(labels), _ptr(row_idx),
                m, n_out, h, v, code,
                int(ignore_index), int(exclude_index), float(logit_softcap),
                _ptr(losses), _ptr(lse), valid_count.data_ptr(),
                ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_forward_dim_first" if in_place else "tlce_forward",
        )
    return losses, lse, valid_count


# ------------------------------------------- forward that leaves the gradients --
def fused_gradients_supported(hidden: torch.Tensor, weight: torch.Tensor,
                              bias: torch.Tensor | None, weight_dim_first: bool) -> bool:
    """Whether ``forward_with_gradients`` takes these operands: bf16 inputs on the
    GPU, head stored [V, H], no bias, H and V multiples of 64.  (f16's exponent
    range cannot hold exp(logit - reference) and its row sums.)"""
    if bias is not None or weight_dim_first or not hidden.is_cuda:
        return False
    if hidden.dtype != torch.bfloat16 or weight.dtype != hidden.dtype:
        return False
    if hidden.dim() != 2 or weight.dim() != 2 or weight.shape[1] != hidden.shape[1]:
        return False
    return bool(_lib.library().tlce_fused_gradients_supported(
        hidden.shape[1], weight.shape[0], _dtype_code(hidden)))


def forward_with_gradients(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
    compute_weight_grad: bool,
    token_weights: torch.Tensor | None = None,
    logit_multiplier: float = 1.0,
    row_idx: torch.Tensor | None = None,
    n_out: int | None = None,
    row_count: torch.Tensor | None = None,
    postpone_weight_grad: bool = False,
):
    """The forward and, in the same pass over the logits, the float32 gradients of
    ``sum_r token_weights[r] * loss[r]`` (three contractions instead of the four
    of ``forward`` + ``backward``).

    Returns ``(losses [n_out] f32, lse [m] f32, valid_count [1] f32,
    grad_hidden_f32 [m, H], grad_weight_f32 [V, H] or None)``;
    ``apply_grad_output`` turns the last two into the gradients of the reduced
    loss once the upstream gradient is known.  ``row_count`` (device int64, with
    ``row_idx``): the real number of rows when the operands are sized for a
    capacity, as the "device" compaction mode leaves them.

    ``postpone_weight_grad`` (with ``compute_weight_grad``, when all rows fit one
    block: ``weight_grad_can_wait``): the grad_weight contraction is left to
    ``grad_weight_from_panel``, which runs it once the upstream gradient is
    known and stores it directly in the input dtype.  The last element returned
    is then the workspace to hand to that call instead of a float32 gradient.
    """
    device = _require_device(hidden, weight, labels, row_idx, token_weights, row_count)
    if not fused_gradients_supported(hidden, weight, None, False):
        raise RuntimeError(
            "forward_with_gradients needs bf16 operands, a [V, H] head and H, V multiples "
            "of 64; use forward / backward for other inputs"
        )
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight.shape[0]
    if labels.numel() != m:
        raise RuntimeError("native linear CE shape mismatch")
    if row_idx is not None and row_idx.numel() != m:
        raise RuntimeError("row_idx must have one entry per row")
    if token_weights is not None:
        token_weights = token_weights.reshape(-1).to(torch.float32).contiguous()
        if token_weights.numel() != m:
            raise RuntimeError("token_weights must have one entry per row")
    n_out = m if n_out is None else int(n_out)
    lib = _lib.library()
    code = _dtype_code(hidden)
    panel = get_panel_bytes()
    with torch.cuda.device(device):
        losses = torch.empty(n_out, dtype=torch.float32, device=device)
        lse = torch.empty(m, dtype=torch.float32, device=device)
        valid_count = torch.empty(1, dtype=torch.float32, device=device)
        grad_hidden32 = torch.empty((m, h), dtype=torch.float32, device=device)
        postpone = bool(postpone_weight_grad and compute_weight_grad)
        if postpone and not weight_grad_can_wait(m, h, v, hidden.dtype):
            raise RuntimeError("the weight gradient can be postponed only when all rows fit "
                               "one block of the forward (weight_grad_can_wait)")
        grad_weight32 = (torch.empty((v, h), dtype=torch.float32, device=device)
                         if compute_weight_grad and not postpone else None)
        ws = _workspace(
            lib.tlce_forward_with_gradients_workspace_bytes(
                m, h, v, code, int(compute_weight_grad), panel),
            device,
        )
        _lib.check(
            lib.tlce_forward_with_gradients(
                _ptr(hidden), _ptr(weight), _ptr(labels), _ptr(row_idx), _ptr(token_weights),
                _ptr(row_count), m, n_out, h, v, code,
                int(ignore_index), int(exclude_index), float(logit_softcap),
                float(logit_multiplier),
                _ptr(losses), _ptr(lse), valid_count.data_ptr(),
                _ptr(grad_hidden32), _ptr(grad_weight32),
                panel, ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_forward_with_gradients",
        )
    return losses, lse, valid_count, grad_hidden32, (ws if postpone else grad_weight32)


def weight_grad_can_wait(m: int, h: int, v: int, dtype: torch.dtype) -> bool:
    """Whether ``forward_with_gradients`` takes ``m`` rows as one block under the
    panel budget in force, so that its grad_weight contraction can be postponed to
    the backward (``grad_weight_from_panel``)."""
    if dtype != torch.bfloat16 or not _lib.library().tlce_fused_gradients_supported(
            h, v, _lib.DTYPE_BF16):
        return False
    return _lib.query_fused_plan(m, h, v, _lib.DTYPE_BF16, get_panel_bytes())["n_blocks"] == 1


def _upstream_gradient(grad_output: torch.Tensor, reduction_code: int, n_out: int) -> torch.Tensor:
    """The upstream gradient as the library reads it: float32, one element for a
    scalar reduction, one per output row for reduction "none"."""
    grad_output = grad_output.reshape(-1).to(torch.float32).contiguous()
    expected = n_out if reduction_code == _lib.REDUCTION_NONE else 1
    if grad_output.numel() != expected:
        raise RuntimeError(f"grad_output has {grad_output.numel()} elements, expected {expected}")
    return grad_output


def grad_weight_from_panel(
    hidden: torch.Tensor,
    workspace: torch.Tensor,
    grad_output: torch.Tensor,
    valid_count: torch.Tensor,
    *,
    reduction: str,
    vocab: int,
    panel_bytes: int,
    row_count: torch.Tensor | None = None,
    row_idx: torch.Tensor | None = None,
    n_out: int | None = None,
) -> torch.Tensor:
    """``grad_weight [V, H]`` in the input dtype from the workspace a
    ``forward_with_gradients(..., postpone_weight_grad=True)`` call left, times the
    upstream gradient (over ``valid_count`` for the mean; for reduction "none" one
    value per output row, ``n_out`` of them, row ``r`` of ``hidden`` taking the one at
    ``row_idx[r]``).  ``panel_bytes`` is the panel budget that forward ran under
    (``get_panel_bytes()`` at that time)."""
    device = _require_device(hidden, workspace, grad_output, valid_count, row_count, row_idx)
    reduction_code = _reduction_code(reduction)
    hidden = _dense(hidden)
    m, h = hidden.shape
    grad_output = _upstream_gradient(grad_output, reduction_code,
                                     m if n_out is None else int(n_out))
    # the C ABI cannot see tensor lengths: what the kernels read must exist
    if row_idx is not None and (row_idx.dtype != torch.long or row_idx.numel() < m):
        raise RuntimeError("row_idx must be int64 with one entry per row of hidden")
    if workspace.dtype != torch.uint8 or not workspace.is_contiguous():
        raise RuntimeError("workspace must be the uint8 buffer forward_with_gradients returned")
    with torch.cuda.device(device):
        grad_weight = torch.empty((int(vocab), h), dtype=hidden.dtype, device=device)
        _lib.check(
            _lib.library().tlce_grad_weight_from_panel(
                _ptr(hidden), _ptr(row_idx), _ptr(row_count), _ptr(grad_output),
                _ptr(valid_count), m, h, int(vocab), _dtype_code(hidden), reduction_code,
                _ptr(grad_weight), int(panel_bytes), workspace.data_ptr(), workspace.numel(),
                _stream(device),
            ),
            "tlce_grad_weight_from_panel",
        )
    return grad_weight


def apply_grad_output(
    grad_hidden32: torch.Tensor,
    grad_weight32: torch.Tensor | None,
    grad_output: torch.Tensor,
    valid_count: torch.Tensor,
    *,
    reduction: str,
    dtype: torch.dtype,
    row_idx: torch.Tensor | None = None,
    n_out: int | None = None,
    vocab: int | None = None,
    row_count: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``(grad_hidden [n_out, H], grad_weight [V, H] or None)`` in ``dtype``: the
    float32 gradients ``forward_with_gradients`` left, times the upstream gradient
    (over ``valid_count`` for the mean), each entry rounded once.  For reduction
    "none" the upstream gradient has one value per output row and only grad_hidden
    can be finished here (``grad_weight32`` must be None: ``grad_weight_from_panel``)."""
    device = _require_device(grad_hidden32, grad_weight32, grad_output, valid_count, row_idx)
    reduction_code = _reduction_code(reduction)
    m, h = grad_hidden32.shape
    v = grad_weight32.shape[0] if grad_weight32 is not None else int(vocab or 1)
    n_out = m if n_out is None else int(n_out)
    grad_output = _upstream_gradient(grad_output, reduction_code, n_out)
    # the C ABI cannot see tensor lengths: what the kernels read must exist
    if grad_hidden32.dtype != torch.float32 or not grad_hidden32.is_contiguous():
        raise RuntimeError("grad_hidden32 must be a contiguous float32 [m, h] tensor")
    if grad_weight32 is not None and (grad_weight32.dtype != torch.float32
                                      or not grad_weight32.is_contiguous()
                                      or grad_weight32.shape[1] != h):
        raise RuntimeError("grad_weight32 must be a contiguous float32 [v, h] tensor")
    if row_idx is not None and (row_idx.dtype != torch.long or row_idx.numel() < m):
        raise RuntimeError("row_idx must be int64 with one entry per row of grad_hidden32")
    if dtype != torch.bfloat16:
        raise RuntimeError("apply_grad_output writes bf16 gradients only")
    code = _lib.DTYPE_BF16
    with torch.cuda.device(device):
        grad_hidden = torch.empty((n_out, h), dtype=dtype, device=device)
        grad_weight = (torch.empty((v, h), dtype=dtype, device=device)
                       if grad_weight32 is not None else None)
        _lib.check(
            _lib.library().tlce_apply_grad_output(
                _ptr(grad_hidden32), _ptr(grad_weight32), _ptr(row_idx), _ptr(row_count),
                _ptr(grad_output), _ptr(valid_count), m, n_out, h, v, code, reduction_code,
                _ptr(grad_hidden), _ptr(grad_weight), _stream(device),
            ),
            "tlce_apply_grad_output",
        )
    return grad_hidden, grad_weight


# ------------------------------------------------------------------- backward --
def _backward(
    hidden, weight, bias, labels, lse, valid_count, grad_output, *,
    reduction, ignore_index, exclude_index, logit_softcap, weight_dim_first,
    compute_weight_grad, row_idx, n_out,
):
    device = _require_device(hidden, weight, bias, labels, lse, valid_count, grad_output, row_idx)
    hidden = _dense(hidden)
    weight_vf, in_place = _head_operand(weight, weight_dim_first)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight_vf.shape[1] if in_place else weight_vf.shape[0]
    n_out = m if n_out is None else int(n_out)
    code = _dtype_code(hidden)
    reduction_code = _reduction_code(reduction)
    grad_output = grad_output.reshape(-1).to(torch.float32).contiguous()
    expected = n_out if reduction_code == _lib.REDUCTION_NONE else 1
    if grad_output.numel() != expected:
        raise RuntimeError(
            f"grad_output has {grad_output.numel()} elements, expected {expected}"
        )
    bias32 = None if bias is None else bias.to(torch.float32).contiguous()
    lib = _lib.library()
    with torch.cuda.device(device):
        grad_hidden = torch.empty((n_out, h), dtype=hidden.dtype, device=device)
        grad_weight = None
        if compute_weight_grad:      # in the layout the library writes: [H, V] in place, else [V, H]
            grad_weight = torch.empty((h, v) if in_place else (v, h), dtype=weight.dtype,
                                      device=device)
        grad_bias32 = (
            torch.empty(v, dtype=torch.float32, device=device) if bias is not None else None
        )
        ws = _workspace(
            lib.tlce_backward_workspace_bytes(
                m, h, v, code, int(compute_weight_grad), int(bias is not None), get_panel_bytes()
            ),
            device,
        )
        entry = lib.tlce_backward_dim_first if in_place else lib.tlce_backward
        _lib.check(
            entry(
                _ptr(hidden), _ptr(weight_vf), _ptr(bias32), _ptr(labels), _ptr(row_idx),
                _ptr(lse), valid_count.data_ptr(), _ptr(grad_output),
                m, n_out, h, v, code,
                reduction_code, int(ignore_index), int(exclude_index), float(logit_softcap),
                _ptr(grad_hidden), _ptr(grad_weight), _ptr(grad_bias32),
                get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_backward_dim_first" if in_place else "tlce_backward",
        )
    if grad_weight is None:
        grad_weight = torch.empty(0, dtype=weight.dtype, device=device)
    elif weight_dim_first and not in_place:
        grad_weight = grad_weight.t().contiguous()
    if grad_bias32 is None:
        grad_bias = torch.empty(0, dtype=torch.float32, device=device)
    else:
        grad_bias = grad_bias32.to(bias.dtype)
    return grad_hidden, grad_weight, grad_bias


def backward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    lse: torch.Tensor,
    valid_count: torch.Tensor,
    grad_output: torch.Tensor,
    *,
    row_block_size: int,
    reduction: str,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
    compute_dtype: torch.dtype,
    weight_dim_first: bool,
    row_idx: torch.Tensor | None = None,
    n_out: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(grad_hidden [n_out, H], grad_weight, grad_bias)`` in the input dtypes."""
    del row_block_size, compute_dtype
    return _backward(
        hidden, weight, bias, labels, lse, valid_count, grad_output,
        reduction=reduction, ignore_index=ignore_index, exclude_index=exclude_index,
        logit_softcap=logit_softcap, weight_dim_first=weight_dim_first,
        compute_weight_grad=True, row_idx=row_idx, n_out=n_out,
    )


def backward_frozen_weight(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    lse: torch.Tensor,
    valid_count: torch.Tensor,
    grad_output: torch.Tensor,
    *,
    row_block_size: int,
    reduction: str,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
    compute_dtype: torch.dtype,
    weight_dim_first: bool,
    row_idx: torch.Tensor | None = None,
    n_out: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """As ``backward`` with the weight-gradient contraction skipped (empty dW)."""
    del row_block_size, compute_dtype
    return _backward(
        hidden, weight, bias, labels, lse, valid_count, grad_output,
        reduction=reduction, ignore_index=ignore_index, exclude_index=exclude_index,
        logit_softcap=logit_softcap, weight_dim_first=weight_dim_first,
        compute_weight_grad=False, row_idx=row_idx, n_out=n_out,
    )


# ---------------------------------------------------------- masked-token loss --
def masked_loss_forward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    token_weights: torch.Tensor | None,
    *,
    m: int | None = None,
    row_idx: torch.Tensor | None = None,
    row_count: torch.Tensor | None = None,
    n_out: int | None = None,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
    logit_multiplier: float = 1.0,
    want_losses: bool = True,
    want_sum: bool = True,
) -> tuple[torch.Tensor | None, torch.Tensor, torch.Tensor, torch.Tensor | None]:
    """The forward with the loss method's arithmetic folded in
    (distributed_block_diffusion_loss, nemotron/model.py:2084-2151): logits
    scaled by ``logit_multiplier`` instead of a scaled copy of ``hidden``, and
    ``weighted_sum = sum_r token_weights[r] * loss_r`` formed on the device.

    ``hidden`` [>= m, H] (vocab-first ``weight`` [V, H]); ``m`` defaults to
    ``hidden.shape[0]``.  With ``row_count`` (device int64 [1]) ``m`` is only the
    capacity: rows past the count carry no loss and the call never synchronises;
    ``hidden`` must then hold ``round_up(m, 64)`` rows (``gather_loss_rows``
    provides them).  Returns ``(losses [n_out] | None, lse [m], valid_count [1],
    weighted_sum [1] | None)``, all float32.
    """
    device = _require_device(hidden, weight, bias, labels, token_weights, row_idx, row_count)
    if hidden.dim() != 2 or weight.dim() != 2 or weight.shape[1] != hidden.shape[1]:
        raise RuntimeError("masked loss expects hidden [N, D] and weight [V, D]")
    if weight.dtype != hidden.dtype:
        raise RuntimeError("native linear CE expects hidden and weight of one dtype")
    if not (want_losses or want_sum):
        raise RuntimeError("masked loss: nothing to compute")
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    h = hidden.shape[1]
    v = weight.shape[0]
    m = hidden.shape[0] if m is None else int(m)
    need_rows = (m + 63) // 64 * 64 if row_count is not None else m
    if hidden.shape[0] < need_rows or labels.numel() < m:
        raise RuntimeError("masked loss: hidden / labels hold fewer rows than m")
    n_out = m if n_out is None else int(n_out)
    bias32 = None if bias is None else bias.to(torch.float32).contiguous()
    if token_weights is not None:
        token_weights = token_weights.reshape(-1).to(torch.float32).contiguous()
        if token_weights.numel() < m:
            raise RuntimeError("masked loss: token_weights holds fewer entries than m")
    lib = _lib.library()
    code = _dtype_code(hidden)
    with torch.cuda.device(device):
        losses = torch.empty(n_out, dtype=torch.float32, device=device) if want_losses else None
        lse = torch.empty(m, dtype=torch.float32, device=device)
        valid_count = torch.empty(1, dtype=torch.float32, device=device)
        weighted_sum = torch.empty(1, dtype=torch.float32, device=device) if want_sum else None
        ws = _workspace(
            lib.tlce_masked_loss_forward_workspace_bytes(m, h, v, code, int(row_count is not None)),
            device,
        )
        _lib.check(
            lib.tlce_masked_loss_forward(
                _ptr(hidden), _ptr(weight), _ptr(bias32), _ptr(labels), _ptr(token_weights),
                _ptr(row_idx), _ptr(row_count), m, n_out, h, v, code,
                int(ignore_index), int(exclude_index), float(logit_softcap),
                float(logit_multiplier),
                _ptr(losses), _ptr(lse), valid_count.data_ptr(), _ptr(weighted_sum),
                ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_masked_loss_forward",
        )
    return losses, lse, valid_count, weighted_sum


def masked_loss_backward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    token_weights: torch.Tensor | None,
    lse: torch.Tensor,
    valid_count: torch.Tensor | None,
    grad_output: torch.Tensor,
    *,
    reduction: str = "sum",
    m: int | None = None,
    row_idx: torch.Tensor | None = None,
    row_count: torch.Tensor | None = None,
    n_out: int | None = None,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
    logit_multiplier: float = 1.0,
    compute_weight_grad: bool = True,
) -> tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None]:
    """Gradients of ``masked_loss_forward``.  ``reduction="sum"`` with
    ``grad_output`` [1] is the gradient of ``weighted_sum``; "none" / "mean" take
    the gradient of the per-token losses / of their mean, as ``backward`` does,
    with ``token_weights`` applied on top.  Returns ``(grad_hidden [n_out, H],
    grad_weight | None, grad_bias | None)`` in the input dtypes."""
    device = _require_device(hidden, weight, bias, labels, token_weights, lse, valid_count,
                             grad_output, row_idx, row_count)
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    h = hidden.shape[1]
    v = weight.shape[0]
    m = hidden.shape[0] if m is None else int(m)
    # the C ABI cannot see tensor lengths: the same row checks as the forward
    need_rows = (m + 63) // 64 * 64 if row_count is not None else m
    if hidden.shape[0] < need_rows or labels.numel() < m or lse.numel() < m:
        raise RuntimeError("masked loss: hidden / labels / lse hold fewer rows than m")
    if weight.dim() != 2 or weight.shape[1] != h or weight.dtype != hidden.dtype:
        raise RuntimeError("masked loss expects weight [V, D] in the dtype of hidden")
    n_out = m if n_out is None else int(n_out)
    code = _dtype_code(hidden)
    reduction_code = _reduction_code(reduction)
    grad_output = grad_output.reshape(-1).to(torch.float32).contiguous()
    expected = n_out if reduction_code == _lib.REDUCTION_NONE else 1
    if grad_output.numel() != expected:
        raise RuntimeError(f"grad_output has {grad_output.numel()} elements, expected {expected}")
    bias32 = None if bias is None else bias.to(torch.float32).contiguous()
    if token_weights is not None:
        token_weights = token_weights.reshape(-1).to(torch.float32).contiguous()
        if token_weights.numel() < m:
            raise RuntimeError("masked loss: token_weights holds fewer entries than m")
    lse = lse.reshape(-1).to(torch.float32).contiguous()
    lib = _lib.library()
    with torch.cuda.device(device):
        grad_hidden = torch.empty((n_out, h), dtype=hidden.dtype, device=device)
        grad_weight = (
            torch.empty((v, h), dtype=weight.dtype, device=device) if compute_weight_grad else None
        )
        grad_bias32 = (
            torch.empty(v, dtype=torch.float32, device=device) if bias is not None else None
        )
        ws = _workspace(
            lib.tlce_backward_workspace_bytes(
                m, h, v, code, int(compute_weight_grad), int(bias is not None), get_panel_bytes()
            ),
            device,
        )
        _lib.check(
            lib.tlce_masked_loss_backward(
                _ptr(hidden), _ptr(weight), _ptr(bias32), _ptr(labels), _ptr(token_weights),
                _ptr(row_idx), _ptr(row_count), _ptr(lse), _ptr(valid_count), _ptr(grad_output),
                m, n_out, h, v, code, reduction_code,
                int(ignore_index), int(exclude_index), float(logit_softcap),
                float(logit_multiplier),
                _ptr(grad_hidden), _ptr(grad_weight), _ptr(grad_bias32),
                get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_masked_loss_backward",
        )
    grad_bias = None if grad_bias32 is None else grad_bias32.to(bias.dtype)
    return grad_hidden, grad_weight, grad_bias


# ------------------------------------------------------------ vocabulary shards --
def vocab_parallel_forward_local(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    *,
    vocab_start: int,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Softmax statistics of one vocabulary shard, without logits storage.

    Same call and results as the reference shim
    (chunked_linear_ce_native.py:185-216): ``weight`` holds the rows
    ``[vocab_start, vocab_start + V_local)`` of the head, ``labels`` and
    ``exclude_index`` are global ids.  Returns ``(local_max, local_sum,
    target_logits, valid_count)``, float32, ``[N]`` each and ``[1]``.
    """
    device = _require_device(hidden, weight, bias, labels)
    if hidden.dim() != 2:
        raise RuntimeError("vocab-parallel hidden must be [N, D]")
    if weight.dim() != 2:
        raise RuntimeError("vocab-parallel weight must be [V_local, D]")
    if weight.shape[1] != hidden.shape[1]:
        raise RuntimeError("vocab-parallel head width mismatch")
    if weight.dtype != hidden.dtype:
        raise RuntimeError("native linear CE expects hidden and weight of one dtype")
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v_local = weight.shape[0]
    if labels.numel() != m:
        raise RuntimeError("vocab-parallel label count mismatch")
    bias32 = None if bias is None else bias.to(torch.float32).contiguous()
    lib = _lib.library()
    code = _dtype_code(hidden)
    with torch.cuda.device(device):
        local_max = torch.empty(m, dtype=torch.float32, device=device)
        local_sum = torch.empty(m, dtype=torch.float32, device=device)
        target_logits = torch.empty(m, dtype=torch.float32, device=device)
        valid_count = torch.empty(1, dtype=torch.float32, device=device)
        ws = _workspace(lib.tlce_forward_workspace_bytes(m, h, v_local, code), device)
        _lib.check(
            lib.tlce_forward_local(
                _ptr(hidden), _ptr(weight), _ptr(bias32), _ptr(labels),
                m, h, v_local, code, int(vocab_start),
                int(ignore_index), int(exclude_index), float(logit_softcap),
                _ptr(local_max), _ptr(local_sum), _ptr(target_logits), valid_count.data_ptr(),
                ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_forward_local",
        )
    return local_max, local_sum, target_logits, valid_count


def vocab_parallel_backward_local(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    labels: torch.Tensor,
    global_lse: torch.Tensor,
    valid_count: torch.Tensor,
    grad_output: torch.Tensor,
    *,
    reduction: str,
    vocab_start: int,
    ignore_index: int,
    exclude_index: int,
    logit_softcap: float,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """One vocabulary shard's exact gradient contributions
    (reference shim, chunked_linear_ce_native.py:218-256): ``grad_hidden`` is
    this shard's partial sum, ``grad_weight`` / ``grad_bias`` cover the shard."""
    device = _require_device(hidden, weight, bias, labels, global_lse, valid_count, grad_output)
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v_local = weight.shape[0]
    code = _dtype_code(hidden)
    reduction_code = _reduction_code(reduction)
    grad_output = grad_output.reshape(-1).to(torch.float32).contiguous()
    expected = m if reduction_code == _lib.REDUCTION_NONE else 1
    if grad_output.numel() != expected:
        raise RuntimeError(
            f"grad_output has {grad_output.numel()} elements, expected {expected}"
        )
    global_lse = global_lse.reshape(-1).to(torch.float32).contiguous()
    bias32 = None if bias is None else bias.to(torch.float32).contiguous()
    lib = _lib.library()
    with torch.cuda.device(device):
        grad_hidden = torch.empty((m, h), dtype=hidden.dtype, device=device)
        grad_weight = torch.empty((v_local, h), dtype=weight.dtype, device=device)
        grad_bias32 = (
            torch.empty(v_local, dtype=torch.float32, device=device) if bias is not None else None
        )
        ws = _workspace(
            lib.tlce_backward_workspace_bytes(
                m, h, v_local, code, 1, int(bias is not None), get_panel_bytes()
            ),
            device,
        )
        _lib.check(
            lib.tlce_backward_local(
                _ptr(hidden), _ptr(weight), _ptr(bias32), _ptr(labels),
                _ptr(global_lse), valid_count.data_ptr(), _ptr(grad_output),
                m, h, v_local, code,
                reduction_code, int(vocab_start), int(ignore_index), int(exclude_index),
                float(logit_softcap),
                _ptr(grad_hidden), _ptr(grad_weight), _ptr(grad_bias32),
                get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_backward_local",
        )
    if grad_bias32 is None:
        grad_bias = torch.empty(0, dtype=torch.float32, device=device)
    else:
        grad_bias = grad_bias32.to(bias.dtype)
    return grad_hidden, grad_weight, grad_bias


# --------------------------------------------------------------- soft embedding --
def soft_embedding(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    *,
    logit_softcap: float,
    embedding_scale: float,
) -> torch.Tensor:
    """``embedding_scale * softmax(cap(hidden @ weight.T)) @ weight`` for
    flattened ``hidden`` [N, H] and ``weight`` [V, H], without a logits buffer."""
    device = _require_device(hidden, weight)
    if hidden.dim() != 2 or weight.dim() != 2 or weight.shape[1] != hidden.shape[1]:
        raise RuntimeError("soft embedding expects hidden [N, H] and weight [V, H]")
    if weight.dtype != hidden.dtype:
        raise RuntimeError("native linear CE expects hidden and weight of one dtype")
    hidden = _dense(hidden)
    weight = _dense(weight)
    m, h = hidden.shape
    v = weight.shape[0]
    code = _dtype_code(hidden)
    lib = _lib.library()
    with torch.cuda.device(device):
        out = torch.empty((m, h), dtype=hidden.dtype, device=device)
        if m == 0:
            return out
        ws = _workspace(lib.tlce_soft_embedding_workspace_bytes(m, h, v, code, get_panel_bytes()), device)
        _lib.check(
            lib.tlce_soft_embedding(
                _ptr(hidden), _ptr(weight), m, h, v, code,
                float(logit_softcap), float(embedding_scale), _ptr(out),
                get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_soft_embedding",
        )
    return out


# -------------------------------------------------------------- frozen-head KL --
def _kl_operands(draft_hidden, draft_weight, teacher_hidden, teacher_weight):
    device = _require_device(draft_hidden, draft_weight, teacher_hidden, teacher_weight)
    tensors = [_dense(t) for t in (draft_hidden, draft_weight, teacher_hidden,
                                        teacher_weight)]
    dh, dw, th, tw = tensors
    if dh.dim() != 2 or th.dim() != 2 or dw.dim() != 2 or tw.dim() != 2:
        raise RuntimeError("DFlash KL expects [tokens, hidden] states and [vocabulary, hidden] heads")
    if dh.shape[0] != th.shape[0] or dw.shape[0] != tw.shape[0]:
        raise RuntimeError("DFlash KL draft and teacher shapes differ")
    if dw.shape[1] != dh.shape[1] or tw.shape[1] != th.shape[1]:
        raise RuntimeError("DFlash KL head width is incompatible")
    if any(t.dtype != dh.dtype for t in tensors):
        raise RuntimeError("DFlash KL tensors must use one dtype")
    return device, dh, dw, th, tw


def dflash_kl_forward(
    draft_hidden: torch.Tensor,
    draft_weight: torch.Tensor,
    teacher_hidden: torch.Tensor,
    teacher_weight: torch.Tensor,
    logit_softcap: float,
    keep_teacher_probabilities: bool = False,
) -> tuple[torch.Tensor, ...]:
    """``(losses, draft_lse, teacher_lse)``, float32 [N]: per-token forward KL
    of the teacher head against the draft head without a logits buffer
    (reference shim, chunked_linear_ce_native.py:259-274).

    ``keep_teacher_probabilities``: also return the teacher probabilities of the
    whole vocabulary (a uint8 buffer, 2 bytes per padded row and vocabulary entry)
    for ``dflash_kl_backward`` to read instead of producing them a second time."""
    device, dh, dw, th, tw = _kl_operands(draft_hidden, draft_weight, teacher_hidden,
                                          teacher_weight)
    m, hd = dh.shape
    ht, v = th.shape[1], dw.shape[0]
    code = _dtype_code(dh)
    lib = _lib.library()
    with torch.cuda.device(device):
        losses = torch.empty(m, dtype=torch.float32, device=device)
        draft_lse = torch.empty(m, dtype=torch.float32, device=device)
        teacher_lse = torch.empty(m, dtype=torch.float32, device=device)
        kept = None
        if m == 0:
            return ((losses, draft_lse, teacher_lse, kept) if keep_teacher_probabilities
                    else (losses, draft_lse, teacher_lse))
        if keep_teacher_probabilities:
            kept = torch.empty(lib.tlce_kl_teacher_probabilities_bytes(m, hd, ht, v, code),
                               dtype=torch.uint8, device=device)
        ws = _workspace(lib.tlce_kl_workspace_bytes(m, hd, ht, v, code, get_panel_bytes()), device)
        _lib.check(
            lib.tlce_kl_forward(
                _ptr(dh), _ptr(dw), _ptr(th), _ptr(tw), m, hd, ht, v, code,
                float(logit_softcap), _ptr(losses), _ptr(draft_lse), _ptr(teacher_lse),
                _ptr(kept), get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_kl_forward",
        )
    if keep_teacher_probabilities:
        return losses, draft_lse, teacher_lse, kept
    return losses, draft_lse, teacher_lse


def kl_gradient_in_forward_supported(draft_hidden, draft_weight, teacher_hidden,
                                     logit_softcap: float) -> bool:
    """Whether ``dflash_kl_forward_with_gradient`` takes these operands (bf16, a soft cap
    between 10 and 40 or none, hidden sizes and V multiples of 64; rows go in blocks of the
    panel budget)."""
    if draft_hidden.dtype != torch.bfloat16 or draft_hidden.shape[0] == 0:
        return False
    return bool(_lib.library().tlce_kl_gradient_in_forward_supported(
        draft_hidden.shape[0], draft_hidden.shape[1], teacher_hidden.shape[1],
        draft_weight.shape[0], _lib.DTYPE_BF16, float(logit_softcap)))


def dflash_kl_forward_with_gradient(
    draft_hidden: torch.Tensor,
    draft_weight: torch.Tensor,
    teacher_hidden: torch.Tensor,
    teacher_weight: torch.Tensor,
    logit_softcap: float,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(losses, draft_lse, teacher_lse, unit)``: ``dflash_kl_forward`` plus
    ``d losses / d draft_hidden`` as a float32 ``[N, D]`` tensor formed in the same
    forward (4 contractions per step); the backward multiplies row ``r`` by its
    upstream gradient (``apply_grad_output(..., reduction="none")``)."""
    device, dh, dw, th, tw = _kl_operands(draft_hidden, draft_weight, teacher_hidden,
                                          teacher_weight)
    m, hd = dh.shape
    ht, v = th.shape[1], dw.shape[0]
    code = _dtype_code(dh)
    lib = _lib.library()
    with torch.cuda.device(device):
        losses = torch.empty(m, dtype=torch.float32, device=device)
        draft_lse = torch.empty(m, dtype=torch.float32, device=device)
        teacher_lse = torch.empty(m, dtype=torch.float32, device=device)
        unit = torch.empty((m, hd), dtype=torch.float32, device=device)
        nbytes = lib.tlce_kl_forward_with_gradient_workspace_bytes(m, hd, ht, v, code,
                                                                    get_panel_bytes())
        if nbytes < 0:
            raise RuntimeError("the KL forward that leaves the gradient does not take these "
                               "operands (kl_gradient_in_forward_supported)")
        ws = _workspace(nbytes, device)
        _lib.check(
            lib.tlce_kl_forward_with_gradient(
                _ptr(dh), _ptr(dw), _ptr(th), _ptr(tw), m, hd, ht, v, code,
                float(logit_softcap), _ptr(losses), _ptr(draft_lse), _ptr(teacher_lse),
                _ptr(unit), get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_kl_forward_with_gradient",
        )
    return losses, draft_lse, teacher_lse, unit


def kl_teacher_probabilities_bytes(draft_hidden, draft_weight, teacher_hidden) -> int:
    """Size of the buffer ``dflash_kl_forward(keep_teacher_probabilities=True)`` fills."""
    m, hd = draft_hidden.shape
    return int(_lib.library().tlce_kl_teacher_probabilities_bytes(
        m, hd, teacher_hidden.shape[1], draft_weight.shape[0], _dtype_code(draft_hidden)))


def dflash_kl_backward(
    draft_hidden: torch.Tensor,
    draft_weight: torch.Tensor,
    teacher_hidden: torch.Tensor,
    teacher_weight: torch.Tensor,
    draft_lse: torch.Tensor,
    teacher_lse: torch.Tensor,
    grad_output: torch.Tensor,
    logit_softcap: float,
    teacher_probabilities: torch.Tensor | None = None,
) -> torch.Tensor:
    """Gradient of the per-token KL with respect to the draft hidden states
    (reference shim, chunked_linear_ce_native.py:277-296).  ``teacher_probabilities``:
    what the forward kept for these operands, or None to produce them again."""
    device, dh, dw, th, tw = _kl_operands(draft_hidden, draft_weight, teacher_hidden,
                                          teacher_weight)
    _require_device(draft_lse, teacher_lse, grad_output)
    m, hd = dh.shape
    ht, v = th.shape[1], dw.shape[0]
    code = _dtype_code(dh)
    grad_output = grad_output.reshape(-1).to(torch.float32).contiguous()
    if grad_output.numel() != m:
        raise RuntimeError(f"grad_output has {grad_output.numel()} elements, expected {m}")
    draft_lse = draft_lse.reshape(-1).to(torch.float32).contiguous()
    teacher_lse = teacher_lse.reshape(-1).to(torch.float32).contiguous()
    lib = _lib.library()
    if teacher_probabilities is not None:
        _require_device(teacher_probabilities)
        need = lib.tlce_kl_teacher_probabilities_bytes(m, hd, ht, v, code)
        if (teacher_probabilities.dtype != torch.uint8 or not teacher_probabilities.is_contiguous()
                or teacher_probabilities.numel() < need):
            raise RuntimeError("teacher_probabilities must be the uint8 buffer the forward kept "
                               f"for these operands ({need} bytes)")
    with torch.cuda.device(device):
        grad_hidden = torch.empty((m, hd), dtype=dh.dtype, device=device)
        if m == 0:
            return grad_hidden
        ws = _workspace(lib.tlce_kl_workspace_bytes(m, hd, ht, v, code, get_panel_bytes()), device)
        _lib.check(
            lib.tlce_kl_backward(
                _ptr(dh), _ptr(dw), _ptr(th), _ptr(tw),
                _ptr(draft_lse), _ptr(teacher_lse), _ptr(grad_output),
                _ptr(teacher_probabilities), m, hd, ht, v, code, float(logit_softcap), _ptr(grad_hidden),
                get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_kl_backward",
        )
    return grad_hidden


# ----------------------------------------------- cross entropy with exact top-k --
def dflash_ce_topk_forward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    top_k: int,
    row_block_size: int,
    output_multiplier: float,
    logit_softcap: float,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(loss, probability, top_values, top_ids, lse)`` of a frozen head
    (reference shim, chunked_linear_ce_native.py:299-319).  ``row_block_size``
    is accepted for signature parity and ignored."""
    del row_block_size
    device = _require_device(hidden, weight, labels)
    if hidden.dim() != 2 or weight.dim() != 2 or weight.shape[1] != hidden.shape[1]:
        raise RuntimeError("CE top-k expects hidden [N, D] and weight [V, D]")
    if weight.dtype != hidden.dtype:
        raise RuntimeError("native linear CE expects hidden and weight of one dtype")
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight.shape[0]
    k = int(top_k)
    code = _dtype_code(hidden)
    lib = _lib.library()
    with torch.cuda.device(device):
        loss = torch.empty(m, dtype=torch.float32, device=device)
        probability = torch.empty(m, dtype=torch.float32, device=device)
        lse = torch.empty(m, dtype=torch.float32, device=device)
        top_values = torch.empty((m, k), dtype=torch.float32, device=device)
        top_ids = torch.empty((m, k), dtype=torch.long, device=device)
        if m:
            ws = _workspace(
                lib.tlce_ce_topk_forward_workspace_bytes(m, h, v, code, get_panel_bytes()), device
            )
            _lib.check(
                lib.tlce_ce_topk_forward(
                    _ptr(hidden), _ptr(weight), _ptr(labels), m, h, v, code, k,
                    float(output_multiplier), float(logit_softcap),
                    _ptr(loss), _ptr(probability), _ptr(top_values), _ptr(top_ids), _ptr(lse),
                    get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
                ),
                "tlce_ce_topk_forward",
            )
    return loss, probability, top_values, top_ids, lse


def ce_topk_gradient_in_forward_supported(hidden: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether ``dflash_ce_topk_forward_with_gradient`` takes these operands: bf16,
    H and V multiples of 64 (rows are taken in blocks of the panel of exponentiated
    logits, 2.5 GiB over the whole vocabulary: 8192 rows at V = 151936)."""
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or hidden.shape[0] == 0:
        return False
    return bool(_lib.library().tlce_ce_topk_gradient_in_forward_supported(
        hidden.shape[0], hidden.shape[1], weight.shape[0], _lib.DTYPE_BF16))


def dflash_ce_topk_forward_with_gradient(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    top_k: int,
    output_multiplier: float,
    logit_softcap: float,
) -> tuple[torch.Tensor, ...]:
    """``dflash_ce_topk_forward`` plus ``d lse / d hidden`` as a float32 ``[N, D]``
    tensor, formed while the forward's logits panels exist (one more contraction
    instead of the backward's two).  ``dflash_ce_topk_apply_gradient`` turns it into
    grad_hidden once the upstream gradients are known."""
    device = _require_device(hidden, weight, labels)
    if hidden.dim() != 2 or weight.dim() != 2 or weight.shape[1] != hidden.shape[1]:
        raise RuntimeError("CE top-k expects hidden [N, D] and weight [V, D]")
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight.shape[0]
    if labels.numel() != m:
        raise RuntimeError("CE top-k expects one label per row")
    k = int(top_k)
    code = _dtype_code(hidden)
    lib = _lib.library()
    with torch.cuda.device(device):
        loss = torch.empty(m, dtype=torch.float32, device=device)
        probability = torch.empty(m, dtype=torch.float32, device=device)
        lse = torch.empty(m, dtype=torch.float32, device=device)
        top_values = torch.empty((m, k), dtype=torch.float32, device=device)
        top_ids = torch.empty((m, k), dtype=torch.long, device=device)
        unit = torch.empty((m, h), dtype=torch.float32, device=device)
        nbytes = lib.tlce_ce_topk_forward_with_gradient_workspace_bytes(m, h, v, code,
                                                                         get_panel_bytes())
        if nbytes < 0:
            raise RuntimeError("CE top-k with the gradient formed in the forward does not take "
                               "these operands (ce_topk_gradient_in_forward_supported)")
        ws = _workspace(nbytes, device)
        _lib.check(
            lib.tlce_ce_topk_forward_with_gradient(
                _ptr(hidden), _ptr(weight), _ptr(labels), m, h, v, code, k,
                float(output_multiplier), float(logit_softcap),
                _ptr(loss), _ptr(probability), _ptr(top_values), _ptr(top_ids), _ptr(lse),
                _ptr(unit), get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
            ),
            "tlce_ce_topk_forward_with_gradient",
        )
    return loss, probability, top_values, top_ids, lse, unit


def dflash_ce_topk_apply_gradient(
    unit: torch.Tensor,
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    probabilities: torch.Tensor,
    top_ids: torch.Tensor,
    grad_loss: torch.Tensor,
    grad_probability: torch.Tensor,
    grad_top_values: torch.Tensor | None,
    *,
    output_multiplier: float,
    logit_softcap: float,
) -> torch.Tensor:
    """grad_hidden from the ``d lse / d hidden`` the forward left: one pass over rows
    that scales it and adds the label's and the top-k ids' single-row terms."""
    device = _require_device(unit, hidden, weight, labels, probabilities, top_ids, grad_loss,
                             grad_probability, grad_top_values)
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight.shape[0]
    k = int(top_ids.shape[1])
    if unit.dtype != torch.float32 or tuple(unit.shape) != (m, h) or not unit.is_contiguous():
        raise RuntimeError("the forward's gradient must be a contiguous float32 [N, D] tensor")
    if labels.numel() != m or top_ids.shape[0] != m:
        raise RuntimeError("CE top-k expects one label and one row of ids per row")
    ce_scale = (grad_loss.float() - grad_probability.float() * probabilities.float()).contiguous()
    gtv = None if grad_top_values is None else grad_top_values.to(torch.float32).contiguous()
    top_ids = top_ids.to(torch.long).contiguous()
    with torch.cuda.device(device):
        grad_hidden = torch.empty((m, h), dtype=hidden.dtype, device=device)
        if m:
            _lib.check(
                _lib.library().tlce_ce_topk_apply_gradient(
                    _ptr(unit), _ptr(hidden), _ptr(weight), _ptr(labels), _ptr(top_ids),
                    _ptr(ce_scale), _ptr(gtv), m, h, v, _dtype_code(hidden), k,
                    float(output_multiplier), float(logit_softcap), _ptr(grad_hidden),
                    _stream(device),
                ),
                "tlce_ce_topk_apply_gradient",
            )
    return grad_hidden


def dflash_ce_topk_backward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    lse: torch.Tensor,
    probabilities: torch.Tensor,
    top_ids: torch.Tensor,
    grad_loss: torch.Tensor,
    grad_probability: torch.Tensor,
    grad_top_values: torch.Tensor | None,
    *,
    row_block_size: int,
    output_multiplier: float,
    logit_softcap: float,
) -> torch.Tensor:
    """Gradient for ``hidden`` given the gradients of loss, probability and
    top values (reference shim, chunked_linear_ce_native.py:322-350)."""
    del row_block_size
    device = _require_device(hidden, weight, labels, lse, probabilities, top_ids, grad_loss,
                             grad_probability, grad_top_values)
    hidden = _dense(hidden)
    weight = _dense(weight)
    labels = labels.reshape(-1).to(torch.long).contiguous()
    m, h = hidden.shape
    v = weight.shape[0]
    k = int(top_ids.shape[1])
    code = _dtype_code(hidden)
    # d objective / d loss, with the probability's gradient folded in (p = exp(-loss))
    ce_scale = (grad_loss.float() - grad_probability.float() * probabilities.float()).contiguous()
    gtv = None if grad_top_values is None else grad_top_values.to(torch.float32).contiguous()
    lse = lse.reshape(-1).to(torch.float32).contiguous()
    top_ids = top_ids.to(torch.long).contiguous()
    lib = _lib.library()
    with torch.cuda.device(device):
        grad_hidden = torch.empty((m, h), dtype=hidden.dtype, device=device)
        if m:
            ws = _workspace(
                lib.tlce_ce_topk_backward_workspace_bytes(m, h, v, code, get_panel_bytes()), device
            )
            _lib.check(
                lib.tlce_ce_topk_backward(
                    _ptr(hidden), _ptr(weight), _ptr(labels), _ptr(lse), _ptr(top_ids),
                    _ptr(ce_scale), _ptr(gtv), m, h, v, code, k,
                    float(output_multiplier), float(logit_softcap), _ptr(grad_hidden),
                    get_panel_bytes(), ws.data_ptr(), ws.numel(), _stream(device),
                ),
                "tlce_ce_topk_backward",
            )
    return grad_hidden
