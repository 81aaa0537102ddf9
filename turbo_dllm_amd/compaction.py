"""Compaction of loss-bearing rows before the LM-head loss.

Counterpart of ``_compact_valid_loss_rows`` and its sibling call-site code
(dllm_parallel/core/models/backbones/nemotron/model.py:4234-4253, :1922-1939,
:2013-2029; dflash/model.py:870-885): keep only rows whose label differs from
``ignore_index``.  On the GPU the indices come from the library's
ballot/prefix-sum kernel and the rows from its gather kernel; gradients flow
back through the matching scatter.  Host tensors use the torch expressions the
reference uses.
"""

from __future__ import annotations

import torch


class _GatherRows(torch.autograd.Function):
    """``src.index_select(0, row_idx)`` through the HIP gather/scatter kernels."""

    @staticmethod
    def forward(ctx, src: torch.Tensor, row_idx: torch.Tensor):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        ctx.save_for_backward(row_idx)
        ctx.n_rows = src.shape[0]
        return native.gather_rows(src, row_idx)

    @staticmethod
    def backward(ctx, grad_out):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        (row_idx,) = ctx.saved_tensors
        # row_idx is strictly ascending, so index_add reduces to a scatter
        return native.scatter_rows(grad_out.contiguous(), row_idx, ctx.n_rows), None


def valid_row_indices(labels: torch.Tensor, ignore_index: int = -100) -> torch.Tensor:
    """Ascending int64 positions of ``labels.reshape(-1) != ignore_index``."""
    flat = labels.reshape(-1)
    if flat.is_cuda:
        from . import chunked_linear_ce_native as native

        row_idx, _ = native.compact_rows(flat, int(ignore_index))
        return row_idx
    return torch.nonzero(flat != int(ignore_index), as_tuple=False).flatten()


def gather_rows(src: torch.Tensor, row_idx: torch.Tensor) -> torch.Tensor:
    """Differentiable row gather; HIP kernels for device tensors."""
    if src.is_cuda:
        return _GatherRows.apply(src.contiguous(), row_idx)
    return src.index_select(0, row_idx)


def compact_valid_loss_rows(
    hidden_states: torch.Tensor,
    labels: torch.Tensor,
    loss_weights: torch.Tensor,
    *,
    ignore_index: int,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Rows of (hidden, labels, float32 weights) whose label is not ``ignore_index``.

    As in the reference, when every row is loss-bearing the hidden states and
    labels are returned as passed (not flattened) and only the weights are
    flattened (nemotron/model.py:4247-4248).
    """
    hidden_2d = hidden_states.reshape(-1, hidden_states.shape[-1])
    labels_1d = labels.reshape(-1)
    weights_1d = loss_weights.reshape(-1).float()
    row_idx = valid_row_indices(labels_1d, ignore_index)
    if row_idx.numel() == labels_1d.numel():
        return hidden_states, labels, weights_1d
    return (
        gather_rows(hidden_2d, row_idx),
        gather_rows(labels_1d, row_idx),
        gather_rows(weights_1d, row_idx),
    )
