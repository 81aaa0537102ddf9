"""Per-token forward KL between two frozen LM heads without a logits buffer.

Same entry point and checks as the reference module
(dllm_parallel/core/kernels/dflash_kl.py:74-121): ``frozen_linear_kl`` returns
``KL(softmax(teacher logits) || softmax(draft logits))`` per token, float32,
and differentiates with respect to the draft hidden states only.  Device
tensors run in the HIP library; host tensors take the dense torch expression.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


# the teacher probabilities kept between forward and backward may take this much
KEPT_TEACHER_BYTES = 5 << 29


class _FrozenLinearKL(torch.autograd.Function):
    """Autograd node around the library's KL forward / backward entry points."""

    @staticmethod
    def forward(ctx, draft_hidden, draft_weight, teacher_hidden, teacher_weight, logit_softcap):
        from . import chunked_linear_ce_native as native

        operands = tuple(t.contiguous() for t in (draft_hidden, draft_weight, teacher_hidden,
                                                  teacher_weight))
        from . import options
        wants = (bool(ctx.needs_input_grad[0]) and options.get_gradient_mode() == "forward"
                 and operands[0].shape[0] > 0)
        # bf16, a soft cap between 10 and 40 or none: the draft
        # pass of the forward leaves what the logit gradient needs, and one contraction
        # more in the forward leaves d loss / d draft_hidden (4 contractions per step);
        # the backward only multiplies each row by its upstream gradient
        ctx.fused = wants and native.kl_gradient_in_forward_supported(
            operands[0], operands[1], operands[2], float(logit_softcap))
        if ctx.fused:
            losses, _, _, unit = native.dflash_kl_forward_with_gradient(*operands,
                                                                        float(logit_softcap))
            ctx.kept = False
            ctx.save_for_backward(unit)
            ctx.grad_dtype = operands[0].dtype
            return losses
        # Otherwise the teacher probabilities of the whole vocabulary stay in memory until
        # the backward when they fit the budget of the other kept panels (2.5 GiB: 8192 rows
        # at V = 151936): the backward then reads them instead of contracting the teacher
        # head a second time (5 contractions per step instead of 6).
        keep = (wants
                and native.kl_teacher_probabilities_bytes(operands[0], operands[1], operands[2])
                <= KEPT_TEACHER_BYTES)
        if keep:
            losses, draft_lse, teacher_lse, kept = native.dflash_kl_forward(
                *operands, float(logit_softcap), keep_teacher_probabilities=True)
        else:
            losses, draft_lse, teacher_lse = native.dflash_kl_forward(*operands,
                                                                      float(logit_softcap))
            kept = None
        ctx.kept = keep
        ctx.save_for_backward(*operands, draft_lse, teacher_lse, *((kept,) if keep else ()))
        ctx.logit_softcap = float(logit_softcap)
        ctx.panel_bytes = native.get_panel_bytes()   # the backward may run on another thread
        return losses

    @staticmethod
    def backward(ctx, grad_output):
        from . import chunked_linear_ce_native as native

        if ctx.fused:
            (unit,) = ctx.saved_tensors
            grad_hidden, _ = native.apply_grad_output(
                unit, None, grad_output.contiguous(), None, reduction="none",
                dtype=ctx.grad_dtype)
            return grad_hidden, None, None, None, None
        saved = list(ctx.saved_tensors)
        kept = saved.pop() if ctx.kept else None
        *operands, draft_lse, teacher_lse = saved
        with native.panel_budget(ctx.panel_bytes):
            grad_hidden = native.dflash_kl_backward(*operands, draft_lse, teacher_lse,
                                                    grad_output.contiguous(), ctx.logit_softcap,
                                                    teacher_probabilities=kept)
        return grad_hidden, None, None, None, None


def _check(draft_hidden, draft_weight, teacher_hidden, teacher_weight, logit_softcap):
    # messages of the reference, dflash_kl.py:84-99
    if draft_hidden.ndim != 2 or teacher_hidden.ndim != 2:
        raise ValueError("DFlash KL hidden states must be [tokens, hidden]")
    if draft_hidden.shape[0] != teacher_hidden.shape[0]:
        raise ValueError("DFlash KL draft and teacher token counts differ")
    if draft_weight.ndim != 2 or teacher_weight.ndim != 2:
        raise ValueError("DFlash KL head weights must be [vocabulary, hidden]")
    if draft_weight.shape[0] != teacher_weight.shape[0]:
        raise ValueError("DFlash KL draft and teacher vocabularies differ")
    if draft_weight.shape[1] != draft_hidden.shape[1]:
        raise ValueError("DFlash KL draft head width is incompatible")
    if teacher_weight.shape[1] != teacher_hidden.shape[1]:
        raise ValueError("DFlash KL teacher head width is incompatible")
    if logit_softcap is not None and logit_softcap <= 0.0:
        raise ValueError("DFlash KL logit_softcap must be positive")


def frozen_linear_kl(
    draft_hidden: torch.Tensor,
    draft_weight: torch.Tensor,
    teacher_hidden: torch.Tensor,
    teacher_weight: torch.Tensor,
    *,
    logit_softcap: float | None = None,
) -> torch.Tensor:
    """Per-token forward KL, float32 [tokens]."""
    _check(draft_hidden, draft_weight, teacher_hidden, teacher_weight, logit_softcap)
    cap = 0.0 if logit_softcap is None else float(logit_softcap)
    others = (draft_weight, teacher_hidden, teacher_weight)
    if draft_hidden.is_cuda:
        if not all(t.is_cuda for t in others):
            raise ValueError("DFlash KL tensors must be on one CUDA device")
        if not all(t.dtype == draft_hidden.dtype for t in others):
            raise ValueError("DFlash KL tensors must use one dtype")
        return _FrozenLinearKL.apply(draft_hidden, draft_weight, teacher_hidden, teacher_weight,
                                     cap)
    if any(t.is_cuda for t in others):
        raise ValueError("DFlash KL tensors must be on one device")
    draft = F.linear(draft_hidden, draft_weight)
    teacher = F.linear(teacher_hidden, teacher_weight)
    if cap > 0.0:
        draft, teacher = (cap * torch.tanh(z / cap) for z in (draft, teacher))
    log_q = F.log_softmax(draft, dim=-1, dtype=torch.float32)
    p = F.softmax(teacher, dim=-1, dtype=torch.float32)
    return F.kl_div(log_q, p, reduction="none").sum(dim=-1)


__all__ = ["frozen_linear_kl"]
