"""Frozen LM-head cross entropy that also returns the exact top-k logits.

Same entry point, checks and outputs as the reference module
(dllm_parallel/core/kernels/dflash_linear_topk.py:228-278):
``frozen_linear_ce_topk`` returns ``(loss, gold probability, top values, top
ids)`` per row without an ``[N, V]`` tensor and differentiates with respect to
``hidden`` through the loss, the probability and the top values.  Device
tensors of 16-bit dtype run in the HIP library; everything else takes a dense
torch path.
"""

from __future__ import annotations

import torch


class _NativeFrozenLinearCETopK(torch.autograd.Function):
    """Autograd node around the library's CE + top-k entry points."""

    @staticmethod
    def forward(ctx, hidden, weight, labels, top_k, output_multiplier, logit_softcap):
        from . import chunked_linear_ce_native as native

        hidden = hidden.contiguous()
        weight = weight.contiguous()
        labels = labels.to(device=hidden.device, dtype=torch.long).contiguous()
        # d lse / d hidden while the forward's logits panels exist (one contraction more
        # in the forward, none in the backward), where the library takes the operands
        from . import options
        ctx.fused = (bool(ctx.needs_input_grad[0]) and options.get_gradient_mode() == "forward"
                     and native.ce_topk_gradient_in_forward_supported(hidden, weight))
        if ctx.fused:
            loss, probability, top_values, top_ids, lse, unit = (
                native.dflash_ce_topk_forward_with_gradient(
                    hidden, weight, labels, top_k=int(top_k),
                    output_multiplier=float(output_multiplier),
                    logit_softcap=float(logit_softcap)))
            ctx.save_for_backward(hidden, weight, labels, unit, probability, top_ids)
            ctx.output_multiplier = float(output_multiplier)
            ctx.logit_softcap = float(logit_softcap)
            ctx.mark_non_differentiable(top_ids)
            return loss, probability, top_values, top_ids
        loss, probability, top_values, top_ids, lse = native.dflash_ce_topk_forward(
            hidden, weight, labels, top_k=int(top_k), row_block_size=0,
            output_multiplier=float(output_multiplier), logit_softcap=float(logit_softcap),
        )
        ctx.save_for_backward(hidden, weight, labels, lse, probability, top_ids)
        ctx.output_multiplier = float(output_multiplier)
        ctx.logit_softcap = float(logit_softcap)
        ctx.panel_bytes = native.get_panel_bytes()   # the backward may run on another thread
        ctx.mark_non_differentiable(top_ids)
        return loss, probability, top_values, top_ids

    @staticmethod
    def backward(ctx, grad_loss, grad_probability, grad_top_values, _grad_top_ids):
        from . import chunked_linear_ce_native as native

        hidden, weight, labels, lse, probability, top_ids = ctx.saved_tensors
        zeros = torch.zeros_like(probability)
        if ctx.fused:
            grad_hidden = native.dflash_ce_topk_apply_gradient(
                lse, hidden, weight, labels, probability, top_ids,   # lse slot: d lse / d hidden
                zeros if grad_loss is None else grad_loss,
                zeros if grad_probability is None else grad_probability,
                grad_top_values,
                output_multiplier=ctx.output_multiplier, logit_softcap=ctx.logit_softcap,
            )
            return grad_hidden, None, None, None, None, None
        with native.panel_budget(ctx.panel_bytes):
            grad_hidden = native.dflash_ce_topk_backward(
                hidden, weight, labels, lse, probability, top_ids,
                zeros if grad_loss is None else grad_loss,
                zeros if grad_probability is None else grad_probability,
                grad_top_values,
                row_block_size=0, output_multiplier=ctx.output_multiplier,
                logit_softcap=ctx.logit_softcap,
            )
        return grad_hidden, None, None, None, None, None


def _dense_ce_topk(hidden, weight, labels, top_k, output_multiplier, logit_softcap):
    """Host / float32 path: plain differentiable torch over the full logits."""
    logits = (hidden @ weight.t()).float() * float(output_multiplier)
    if logit_softcap > 0:
        logits = torch.tanh(logits / logit_softcap) * logit_softcap
    lse = torch.logsumexp(logits, dim=-1)
    loss = lse - logits.gather(1, labels.to(torch.long)[:, None])[:, 0]
    top_values, top_ids = logits.topk(int(top_k), dim=-1)
    return loss, torch.exp(-loss), top_values, top_ids


def frozen_linear_ce_topk(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    top_k: int,
    vocab_block_size: int = 32768,
    output_multiplier: float = 1.0,
    logit_softcap: float | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """CE, gold probability and exact top-k without an ``[N, V]`` tensor."""
    # checks and messages of the reference, dflash_linear_topk.py:241-258
    if hidden.ndim != 2 or weight.ndim != 2 or labels.ndim != 1:
        raise ValueError("frozen_linear_ce_topk expects [N,D], [V,D], and [N]")
    if hidden.shape[0] != labels.shape[0] or hidden.shape[1] != weight.shape[1]:
        raise ValueError("frozen_linear_ce_topk tensor dimensions are incompatible")
    if weight.requires_grad:
        raise ValueError("frozen_linear_ce_topk requires a frozen weight")
    if not 0 < int(top_k) <= int(weight.shape[0]):
        raise ValueError("top_k must be in the vocabulary range")
    if labels.numel() and (int(labels.min()) < 0 or int(labels.max()) >= weight.shape[0]):
        raise ValueError("labels are outside the vocabulary")
    softcap = 0.0 if logit_softcap is None else float(logit_softcap)
    if logit_softcap is not None and softcap <= 0:
        raise ValueError("logit_softcap must be positive")
    del vocab_block_size   # bounds the reference's torch temporaries only
    native = (hidden.is_cuda and hidden.dtype in {torch.float16, torch.bfloat16}
              and int(top_k) <= 256)
    if native:
        return _NativeFrozenLinearCETopK.apply(hidden, weight, labels, int(top_k),
                                               float(output_multiplier), softcap)
    return _dense_ce_topk(hidden, weight, labels, int(top_k), float(output_multiplier), softcap)


__all__ = ["frozen_linear_ce_topk"]
