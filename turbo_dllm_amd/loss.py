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

from .compaction import compact_valid_loss_rows, gather_rows
from .options import get_gradient_mode, resolve_compaction
from .tiled_linear_cross_entropy import tiled_linear_cross_entropy

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

        rows, targets, token_weights, row_idx, row_count, m = native.compact_loss_rows(
            hidden_flat, labels_flat, weights_flat, -100, mode)
        # gradients while the logits exist (3 contractions instead of 4), where the
        # library takes the operands and the row count is known to the host
        ctx.fused = (
            bool(ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
            and get_gradient_mode() == "forward"
            and native.fused_gradients_supported(rows, weight, bias, False)
        )
        if ctx.fused:
            rows = rows[:m]
            ctx.postponed = bool(ctx.needs_input_grad[1]) and native.weight_grad_can_wait(
                m, rows.shape[1], weight.shape[0], rows.dtype)
            losses, _, valid_count, grad_rows32, grad_weight32 = native.forward_with_gradients(
                rows, weight, targets[:m], ignore_index=-100, exclude_index=exclude_index,
                logit_softcap=logit_softcap, compute_weight_grad=bool(ctx.needs_input_grad[1]),
                token_weights=None if token_weights is None else token_weights[:m],
                logit_multiplier=multiplier,
                row_idx=row_idx, n_out=n, row_count=row_count if mode == "device" else None,
                postpone_weight_grad=ctx.postponed,
            )
            ctx.save_for_backward(grad_rows32, grad_weight32, valid_count, row_idx,
                                  row_count if mode == "device" else None,
                                  rows if ctx.postponed else None)
            ctx.panel_bytes = native.get_panel_bytes()
            ctx.hidden_shape = hidden.shape
            ctx.n_rows, ctx.m = n, m
            ctx.grad_dtype, ctx.vocab = hidden.dtype, weight.shape[0]
            # losses holds the unweighted token losses at their positions, zeros elsewhere
            return torch.dot(losses, weights_flat)
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
        ctx.panel_bytes = native.get_panel_bytes()   # the backward may run on another thread
        return weighted_sum.reshape(())

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        if ctx.fused:
            grad_rows32, grad_weight32, valid_count, row_idx, row_count, rows = ctx.saved_tensors
            grad_hidden, grad_weight = native.apply_grad_output(
                grad_rows32, None if ctx.postponed else grad_weight32, grad_output, valid_count,
                reduction="sum", dtype=ctx.grad_dtype, row_idx=row_idx, n_out=ctx.n_rows,
                vocab=ctx.vocab, row_count=row_count,
            )
            if ctx.postponed:
                grad_weight = native.grad_weight_from_panel(
                    rows, grad_weight32, grad_output, valid_count, reduction="sum",
                    vocab=ctx.vocab, panel_bytes=ctx.panel_bytes, row_count=row_count,
                )
            return (grad_hidden.reshape(ctx.hidden_shape), grad_weight, None) + (None,) * 6
        rows, weight, bias, targets, token_weights, lse, row_idx, row_count = ctx.saved_tensors
        with native.panel_budget(ctx.panel_bytes):
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
        ctx.panel_bytes = native.get_panel_bytes()
        return losses.reshape(labels.shape)

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        rows, weight, bias, targets, lse, valid_count = ctx.saved_tensors
        with native.panel_budget(ctx.panel_bytes):
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
    compaction: Optional[str] = None,
) -> torch.Tensor:
    """Weighted masked-token cross entropy of ``output_head`` on ``hidden``.

    ``hidden`` is [..., H], ``labels`` and ``loss_weights`` share its leading
    shape; labels equal to -100 carry no loss.  ``output_head`` is any module
    with a ``weight`` [V, H] (and optional ``bias``), e.g. ``VocabParallelLinear``
    or ``nn.Linear``, or a module that only offers ``parallel_cross_entropy``.

    Device tensors with a linear head take the fused path (see the module
    docstring); how it compacts rows follows ``compaction`` ("sync", "device" or
    "none") or, when that is None, the calling context's
    ``options.compaction_mode``.  Host tensors, and heads
    without a weight matrix, take the reference's sequence of calls.
    """
    excluded = int(mask_token_id) if (exclude_mask_token and mask_token_id is not None) else None
    weight = getattr(output_head, "weight", None)
    bias = getattr(output_head, "bias", None)
    bias = bias if isinstance(bias, torch.Tensor) else None
    multiplier = 1.0 if output_multiplier is None else float(output_multiplier)
    if isinstance(weight, torch.Tensor) and weight.dim() == 2 and _fused_path_applies(
            hidden, weight, bias, labels, multiplier, loss_weights):
        mode = resolve_compaction(compaction)
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


# ------------------------------------------------------------ DFlash loss method --
class _SegmentWeightedSum(torch.autograd.Function):
    """``out[s] = sum_r values[r] * weights[r]`` over the compacted rows of sample
    ``s``, in a fixed order on the device (the reference's ``scatter_add_`` of the
    per-token losses into per-sample numerators, dflash/model.py:925-937)."""

    @staticmethod
    def forward(ctx, values, weights, row_idx, segment_length, n_segments):  # type: ignore[override]
        from . import chunked_linear_ce_native as native

        ctx.save_for_backward(weights, row_idx)
        ctx.segment_length = int(segment_length)
        return native.segment_weighted_sum(values, weights, row_idx, segment_length, n_segments)

    @staticmethod
    def backward(ctx, grad_out):  # type: ignore[override]
        weights, row_idx = ctx.saved_tensors
        sample = torch.div(row_idx, ctx.segment_length, rounding_mode="floor")
        return grad_out.index_select(0, sample) * weights, None, None, None, None


def dflash_token_loss(
    hidden_states: torch.Tensor,
    target_token_ids: torch.Tensor,
    supervised_mask: torch.Tensor,
    position_weights: torch.Tensor,
    lm_head: nn.Module,
    *,
    loss_kind: str,
    normalization_count: torch.Tensor,
    loss_scale: float = 1.0,
    logit_softcap: Optional[float] = None,
    teacher_hidden_states: Optional[torch.Tensor] = None,
    teacher_head: Optional[nn.Module] = None,
    teacher_norm: Optional[nn.Module] = None,
) -> torch.Tensor:
    """The DFlash drafter loss over the supervised positions of a ``[B, T]`` batch:

        loss = mean_b( sum_{r in sample b} token_loss_r * w_r / (count_b + 1e-5) ) * loss_scale

    One-GPU counterpart of ``distributed_dflash_loss``
    (dllm_parallel/core/models/backbones/dflash/model.py:862-960).
    ``hidden_states`` [B, T, H], ``target_token_ids`` / ``supervised_mask`` (bool) /
    ``position_weights`` [B, T], ``normalization_count`` [B].  ``loss_kind``:

      "paper_ce"        cross entropy of ``lm_head`` against the target tokens
                        (``tiled_linear_cross_entropy``, reduction "none");
      "speculators_kl"  forward KL of the frozen teacher head against the frozen draft
                        head (``frozen_linear_kl``) on ``teacher_norm(teacher rows)``.

    On the GPU the mask is scanned by the library's ballot / prefix-sum kernel,
    rows are gathered by its gather kernel, and the per-sample numerators are
    summed in a fixed order by one workgroup per sample (no ``scatter_add_``
    atomics).  A batch with no supervised position returns a zero that keeps
    the graph of ``hidden_states`` and ``lm_head`` alive, as the reference does.
    """
    from .dflash_kl import frozen_linear_kl

    if loss_kind not in ("paper_ce", "speculators_kl"):
        raise ValueError(f"unsupported DFlash loss {loss_kind!r}")
    if supervised_mask.dim() != 2:
        raise ValueError("DFlash supervised mask must be [batch, tokens]")
    batch_size, tokens_per_sample = (int(x) for x in supervised_mask.shape)
    hidden_flat = hidden_states.reshape(-1, hidden_states.shape[-1])
    device_path = hidden_states.is_cuda
    if device_path:
        from . import chunked_linear_ce_native as native

        valid_indices, n_valid = native.compact_mask(supervised_mask)
    else:
        valid_indices = torch.nonzero(supervised_mask.reshape(-1), as_tuple=False).flatten()
        n_valid = valid_indices.numel()

    denominators = normalization_count.to(device=hidden_states.device, dtype=torch.float32)
    if tuple(denominators.shape) != (batch_size,):
        raise ValueError("DFlash normalization count must contain one value per sample")

    if n_valid == 0:
        # numerators are all zero: only the dependence on the parameters remains
        zero = zero_loss_with_module_parameters(hidden_states, lm_head)
        numerators = zero.reshape(1).expand(batch_size) * 1.0
    else:
        hidden = gather_rows(hidden_flat, valid_indices)
        weights = gather_rows(position_weights.reshape(-1).contiguous(),
                              valid_indices).to(torch.float32)
        if loss_kind == "speculators_kl":
            if teacher_hidden_states is None or teacher_head is None:
                raise RuntimeError("DFlash KL requires teacher logits")
            with torch.no_grad():
                teacher_hidden = gather_rows(
                    teacher_hidden_states.reshape(-1, teacher_hidden_states.shape[-1]),
                    valid_indices)
                if teacher_norm is not None:
                    teacher_hidden = teacher_norm(teacher_hidden)
            token_loss = frozen_linear_kl(hidden, lm_head.weight, teacher_hidden,
                                          teacher_head.weight, logit_softcap=logit_softcap)
        else:
            targets = gather_rows(target_token_ids.reshape(-1).contiguous(), valid_indices)
            if (device_path and get_gradient_mode() == "forward"
                    and (hidden.requires_grad or lm_head.weight.requires_grad)
                    and native.fused_gradients_supported(hidden, lm_head.weight, None, False)):
                # The whole reduction is linear in the token losses,
                #   loss = sum_r token_loss_r * w_r / ((count_{b(r)} + 1e-5) * B),
                # and its per-row factors depend on the inputs only, so the gradients can
                # be formed while the logits exist (three contractions instead of four; two
                # instead of three with a frozen head) and the upstream gradient is a scalar.
                sample = torch.div(valid_indices, tokens_per_sample, rounding_mode="floor")
                row_factors = weights / ((denominators[sample] + 1.0e-5) * batch_size)
                loss = _FusedMaskedTokenLoss.apply(
                    hidden, lm_head.weight, None, targets, row_factors, 1.0, -1,
                    0.0 if logit_softcap is None else float(logit_softcap), "none")
                return loss * float(loss_scale)
            # the rows are compacted and every one of them bears loss
            token_loss = tiled_linear_cross_entropy(
                hidden, lm_head.weight, targets, reduction="none", dtype=hidden.dtype,
                weight_layout="vocab_first", logit_softcap=logit_softcap, compaction="none")
        if device_path:
            numerators = _SegmentWeightedSum.apply(token_loss.float(), weights, valid_indices,
                                                   tokens_per_sample, batch_size)
        else:
            sample_indices = torch.div(valid_indices, tokens_per_sample, rounding_mode="floor")
            numerators = torch.zeros(batch_size, dtype=torch.float32, device=token_loss.device)
            numerators = numerators.scatter_add(0, sample_indices, token_loss.float() * weights)
    loss = (numerators / (denominators + 1.0e-5)).mean()
    return loss * float(loss_scale)
