"""Masked-token loss wrapper around the fused linear cross entropy.

One-GPU counterpart of the reference's block-diffusion loss method
(``distributed_block_diffusion_loss``,
dllm_parallel/core/models/backbones/nemotron/model.py:2046-2151) and of
``zero_loss_with_module_parameters`` (dllm_parallel/core/models/loss.py:13-31):

    loss = sum_r( CE_r * weight_r ) / valid_token_count * loss_scale

over the rows whose label is not -100, with the hidden states optionally
multiplied by ``output_multiplier`` first and the mask token optionally
removed from the softmax.  Only the reduction arithmetic lives here; the
projection, softmax and their gradients run in the HIP library.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from .compaction import compact_valid_loss_rows
from .tiled_linear_cross_entropy import tiled_linear_cross_entropy


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
    shape; labels equal to -100 carry no loss.  ``output_head`` is either a
    module with ``parallel_cross_entropy`` (``VocabParallelLinear``) or any
    module with a ``weight`` [V, H] (and optional ``bias``).
    """
    rows, targets, weights = compact_valid_loss_rows(
        hidden, labels, loss_weights, ignore_index=-100
    )
    if output_multiplier is not None:
        rows = rows * float(output_multiplier)
    if targets.numel() == 0:
        return zero_loss_with_module_parameters(rows, output_head) / valid_token_count * float(
            loss_scale
        )
    excluded = int(mask_token_id) if (exclude_mask_token and mask_token_id is not None) else None
    parallel_ce = getattr(output_head, "parallel_cross_entropy", None)
    if callable(parallel_ce):
        token_losses = parallel_ce(
            rows, targets, ignore_index=-100, exclude_index=excluded, reduction="none",
            logit_softcap=logit_softcap,
        )
    else:
        weight = getattr(output_head, "weight", None)
        if not isinstance(weight, torch.Tensor):
            raise RuntimeError("masked_token_loss requires a linear output head")
        bias = getattr(output_head, "bias", None)
        token_losses = tiled_linear_cross_entropy(
            rows, weight, targets,
            bias=bias if isinstance(bias, torch.Tensor) else None,
            reduction="none", ignore_index=-100, exclude_index=excluded,
            logit_softcap=logit_softcap, dtype=rows.dtype, weight_layout="vocab_first",
        )
    loss_sum = (token_losses.reshape(-1).float() * weights).sum()
    return loss_sum / valid_token_count * float(loss_scale)
