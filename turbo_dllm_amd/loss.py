"""Masked-token loss around the fused linear cross entropy.

One-GPU counterpart of the reference's block-diffusion loss method
(``distributed_block_diffusion_loss``,
dllm_parallel/core/models/backbones/nemotron/model.py:2046-2151) and of
``zero_loss_with_module_parameters`` (dllm_parallel/core/models/loss.py:13-31):

    loss = sum_r( CE_r * weight_r ) / valid_token_count * loss_scale

over the rows whose label is not -100, with the logits optionally multiplied
by ``output_multiplier`` and the mask token optionally removed from the
softmax.

On the GPU the wrapper's arithmetic is folded into the HIP kernels: the
multiplier scales the logits inside the kernels instead of a copy of the
hidden states, the per-token weights enter the kernels' per-row scale vector,
the weighted sum is formed on the device, and rows are compacted once (one
fused gather of hidden rows, labels and weights).  What remains in torch are
two scalar operations (``/ valid_token_count * loss_scale``), whose gradient
reaches the kernels through the scalar ``grad_output``.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from .compaction import compact_valid_loss_rows
from .tiled_linear_cross_entropy import get_compaction_mode, tiled_linear_cross_entropy

_DEVICE_DTYPES = (torch.float16, torch.bfloat16, torch.float32)


def zero_loss_with_module_parameters(hidden_states: torch.Tensor, module: nn.Module) -> torch.Tensor:
    """Exact zero that still depends on ``hidden_states`` and every trainable
    parameter of ``module`` (a rank with no supervised token keeps its graph)."""
    if hidden_states.numel() == 0:
        loss = hidden_states.sum(dtype=torch.float32) * 0.0
    else:
        loss = hidden_states.reshape(-1)[0].float() * 0.0
    for parameter in module.parameters():
        if parameter.requires_grad and parameter.numel() > 0:
            loss = loss + parameter.reshape(-1)[0].float() * 0.0
    return loss


class _FusedMaskedTokenLoss(torch.autograd.Function):
    """``sum_r weight_r * CE_r`` of a linear head over the loss-bearing rows:
    compaction, fused gather, forward and backward all in the HIP library."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels, loss_weights, multiplier, exclude_index,
                logit_softcap, mode):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        hidden_flat = hidden.reshape(-1, hidden.shape[-1]).contiguous()
        labels_flat = labels.reshape(-1).to(torch.long).contiguous()
        weights_flat = loss_weights.reshape(-1).to(torch.float32).contiguous()
        weight = weight.contiguous()
        n = hidden_flat.shape[0]

        row_idx = row_count = None
        rows, targets, token_weights, m = hidden_flat, labels_flat, weights_flat, n
        if mode == "sync":
            row_idx, m = native.compact_rows(labels_flat, -100)
            if m == n:
                row_idx = None
            else:
                rows = native.gather_rows(hidden_flat, row_idx)
                targets = native.gather_rows(labels_flat, row_idx)
                token_weights = native.gather_rows(weights_flat, row_idx)
        elif mode == "device":
            row_idx, row_count = native.compact_rows_device(labels_flat, -100)
            rows, targets, token_weights = native.gather_loss_rows(
                hidden_flat, labels_flat, weights_flat, row_idx, row_count, -100)
        _, lse, _, weighted_sum = native.masked_loss_forward(
            rows, weight, bias, targets, token_weights, m=m, row_idx=row_idx,
            row_count=row_count, n_out=n, ignore_index=-100, exclude_index=exclude_index,
            logit_softcap=logit_softcap, logit_multiplier=multiplier,
            want_losses=False, want_sum=True,
        )
        ctx.save_for_backward(rows, weight, bias, targets, token_weights, lse, row_idx, row_count)
        ctx.hidden_shape = hidden.shape
        ctx.n_rows, ctx.m = n, m
        ctx.multiplier, ctx.exclude_index, ctx.logit_softcap = multiplier, exclude_index, logit_softcap
        return weighted_sum.reshape(())

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        rows, weight, bias, targets, token_weights, lse, row_idx, row_count = ctx.saved_tensors
        grad_hidden, grad_weight, grad_bias = native.masked_loss_backward(
            rows, weight, bias, targets, token_weights, lse, None, grad_output,
            reduction="sum", m=ctx.m, row_idx=row_idx, row_count=row_count, n_out=ctx.n_rows,
            ignore_index=-100, exclude_index=ctx.exclude_index,
            logit_softcap=ctx.logit_softcap, logit_multiplier=ctx.multiplier,
            compute_weight_grad=ctx.needs_input_grad[1],
        )
        return (
            grad_hidden.reshape(ctx.hidden_shape),
            grad_weight if ctx.needs_input_grad[1] else None,
            grad_bias if (bias is not None and ctx.needs_input_grad[2]) else None,
        ) + (None,) * 6


class _FusedTokenLosses(torch.autograd.Function):
    """Per-token CE of a linear head with the output multiplier folded into the
    kernels; rows are taken as given (the callers have compacted them)."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels, multiplier, logit_softcap):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        rows = hidden.reshape(-1, hidden.shape[-1]).contiguous()
        targets = labels.reshape(-1).to(torch.long).contiguous()
        weight = weight.contiguous()
        losses, lse, valid_count, _ = native.masked_loss_forward(
            rows, weight, bias, targets, None, ignore_index=-100, exclude_index=-1,
            logit_softcap=logit_softcap, logit_multiplier=multiplier,
            want_losses=True, want_sum=False,
        )
        ctx.save_for_backward(rows, weight, bias, targets, lse, valid_count)
        ctx.hidden_shape = hidden.shape
        ctx.multiplier, ctx.logit_softcap = multiplier, logit_softcap
        return losses.reshape(labels.shape)

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        rows, weight, bias, targets, lse, valid_count = ctx.saved_tensors
        grad_hidden, grad_weight, grad_bias = native.masked_loss_backward(
            rows, weight, bias, targets, None, lse, valid_count, grad_output,
            reduction="none", ignore_index=-100, exclude_index=-1,
            logit_softcap=ctx.logit_softcap, logit_multiplier=ctx.multiplier,
            compute_weight_grad=ctx.needs_input_grad[1],
        )
        return (
            grad_hidden.reshape(ctx.hidden_shape),
            grad_weight if ctx.needs_input_grad[1] else None,
            grad_bias if (bias is not None and ctx.needs_input_grad[2]) else None,
            None, None, None,
        )


def _fused_path_applies(hidden, weight, bias, labels, multiplier, loss_weights=None) -> bool:
    if not (hidden.is_cuda and weight.is_cuda and labels.is_cuda):
        return False
    if loss_weights is not None and (not loss_weights.is_cuda or loss_weights.requires_grad):
        return False   # the fused path forms no gradient for the weights
    if hidden.dtype not in _DEVICE_DTYPES or weight.dtype != hidden.dtype:
        return False
    if bias is not None and (not bias.is_cuda or bias.dtype != hidden.dtype):
        return False
    return multiplier > 0.0    # the kernels keep a running maximum of the unscaled logits


def masked_token_loss(
    hidden: torch.Tensor,
    labels: torch.Tensor,
    loss_weights: torch.Tensor,
    output_head: nn.Module,
    *,
    valid_token_count: float | torch.Tensor,
    mask_token_id: Optional[int] = None,
    exclude_mask_token: bool = True,
    output_multiplier: Optional[float] = None,
    logit_softcap: Optional[float] = None,
    loss_scale: float = 1.0,
) -> torch.Tensor:
    """Weighted masked-token cross entropy of ``output_head`` on ``hidden``.

    ``hidden`` is [..., H], ``labels`` and ``loss_weights`` share its leading
    shape; labels equal to -100 carry no loss.  ``output_head`` is any module
    with a ``weight`` [V, H] (and optional ``bias``), e.g. ``VocabParallelLinear``
    or ``nn.Linear``, or a module that only offers ``parallel_cross_entropy``.

    Device tensors with a linear head take the fused path (see the module
    docstring); how it compacts rows follows
    ``tiled_linear_cross_entropy.set_compaction_mode``.  Host tensors, and heads
    without a weight matrix, take the reference's sequence of calls.
    """
    excluded = int(mask_token_id) if (exclude_mask_token and mask_token_id is not None) else None
    weight = getattr(output_head, "weight", None)
    bias = getattr(output_head, "bias", None)
    bias = bias if isinstance(bias, torch.Tensor) else None
    multiplier = 1.0 if output_multiplier is None else float(output_multiplier)
    if isinstance(weight, torch.Tensor) and weight.dim() == 2 and _fused_path_applies(
            hidden, weight, bias, labels, multiplier, loss_weights):
        mode = get_compaction_mode()
        if mode == "sync" and labels.numel() == 0:
            return zero_loss_with_module_parameters(hidden, output_head) / valid_token_count * float(
                loss_scale)
        loss_sum = _FusedMaskedTokenLoss.apply(
            hidden, weight, bias, labels, loss_weights, multiplier,
            -1 if excluded is None else excluded,
            0.0 if logit_softcap is None else float(logit_softcap), mode,
        )
        return loss_sum / valid_token_count * float(loss_scale)

    rows, targets, weights = compact_valid_loss_rows(
        hidden, labels, loss_weights, ignore_index=-100
    )
    if output_multiplier is not None:
        rows = rows * float(output_multiplier)
    if targets.numel() == 0:
        return zero_loss_with_module_parameters(rows, output_head) / valid_token_count * float(
            loss_scale
        )
    parallel_ce = getattr(output_head, "parallel_cross_entropy", None)
    if callable(parallel_ce):
        token_losses = parallel_ce(
            rows, targets, ignore_index=-100, exclude_index=excluded, reduction="none",
            logit_softcap=logit_softcap,
        )
    else:
        if not isinstance(weight, torch.Tensor):
            raise RuntimeError("masked_token_loss requires a linear output head")
        token_losses = tiled_linear_cross_entropy(
            rows, weight, targets, bias=bias,
            reduction="none", ignore_index=-100, exclude_index=excluded,
            logit_softcap=logit_softcap, dtype=rows.dtype, weight_layout="vocab_first",
        )
    loss_sum = (token_losses.reshape(-1).float() * weights).sum()
    return loss_sum / valid_token_count * float(loss_scale)


def native_token_cross_entropy(
    hidden_states: torch.Tensor,
    labels: torch.Tensor,
    output_head: nn.Module,
    *,
    output_multiplier: Optional[float] = None,
    logit_softcap: Optional[float] = None,
) -> torch.Tensor:
    """Per-token cross entropy of ``output_head`` on rows the caller has already
    compacted, float32 and shaped like ``labels``: the reference's
    ``_native_token_cross_entropy`` (nemotron/model.py:1866-1902).  On the GPU the
    output multiplier scales the logits inside the kernels; no scaled copy of
    the hidden states is made."""
    weight = getattr(output_head, "weight", None)
    bias = getattr(output_head, "bias", None)
    bias = bias if isinstance(bias, torch.Tensor) else None
    multiplier = 1.0 if output_multiplier is None else float(output_multiplier)
    if isinstance(weight, torch.Tensor) and weight.dim() == 2 and _fused_path_applies(
            hidden_states, weight, bias, labels, multiplier) and labels.numel() > 0:
        return _FusedTokenLosses.apply(
            hidden_states, weight, bias, labels, multiplier,
            0.0 if logit_softcap is None else float(logit_softcap),
        )
    if output_multiplier is not None:
        hidden_states = hidden_states * float(output_multiplier)
    parallel_ce = getattr(output_head, "parallel_cross_entropy", None)
    if callable(parallel_ce):
        losses = parallel_ce(
            hidden_states, labels, ignore_index=-100, exclude_index=None, reduction="none",
            logit_softcap=logit_softcap,
        )
    else:
        if not isinstance(weight, torch.Tensor):
            raise RuntimeError("native DiffusionGemma requires a linear output head")
        losses = tiled_linear_cross_entropy(
            hidden_states, weight, labels, bias=bias, reduction="none", ignore_index=-100,
            exclude_index=None, logit_softcap=logit_softcap, dtype=hidden_states.dtype,
            weight_layout="vocab_first",
        )
    return losses.reshape(labels.shape).float()
