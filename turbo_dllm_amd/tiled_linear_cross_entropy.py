"""LM-head projection + masked-token cross entropy without [N, V] logits.

Drop-in for the reference loss API
``dllm_parallel.core.kernels.tiled_linear_cross_entropy.tiled_linear_cross_entropy``
(dllm_parallel/core/kernels/tiled_linear_cross_entropy.py:459-551): same name,
keywords, return shapes/dtypes, reductions and error behaviour.

Dispatch (tiled_linear_cross_entropy.py:506-551 of the reference):
  * device tensors  -> the gfx950 HIP library (chunked_linear_ce_native); the
    loss-bearing rows are first compacted on the device (ballot + prefix-sum
    kernel), so rows whose label is ``ignore_index`` cost no GEMM work;
  * host tensors    -> ``_HostTiledLinearCrossEntropy``, a pure-torch vocabulary
    streaming implementation (the reference API accepts CPU tensors too);
  * mixed devices   -> RuntimeError.  A device call never falls back to the
    host implementation.

Semantics that differ between the reference's own two paths are resolved in
favour of its native (CUDA) path: the excluded vocabulary column is removed
from the softmax outright, also under a soft cap
(fused_linear_ce_cuda.cu:181-183, 201-203, 270).
"""

from __future__ import annotations

from typing import Optional

import torch

from . import options
from .options import (COMPACTION_MODES, compaction_mode, get_compaction_mode,  # noqa: F401
                      resolve_compaction, set_compaction_mode)


def _canonical_dtype(dtype: torch.dtype | str) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        return dtype
    names = {
        "float32": torch.float32,
        "float64": torch.float64,
        "bfloat16": torch.bfloat16,
        "float16": torch.float16,
    }
    if dtype in names:
        return names[dtype]
    raise ValueError(f"Unsupported dtype: {dtype}")


def _infer_weight_layout(hidden_dim: int, weight: torch.Tensor, weight_layout: str) -> bool:
    """True when ``weight`` is [D, V] (dim-first), False when it is [V, D]."""
    if weight_layout not in {"auto", "vocab_first", "dim_first"}:
        raise ValueError("weight_layout must be one of 'auto', 'vocab_first', or 'dim_first'")
    shape = tuple(weight.shape)
    if weight_layout == "vocab_first":
        if weight.ndim != 2 or shape[1] != hidden_dim:
            raise ValueError(f"Expected vocab-first weight [V, {hidden_dim}], got {shape}")
        return False
    if weight_layout == "dim_first":
        if weight.ndim != 2 or shape[0] != hidden_dim:
            raise ValueError(f"Expected dim-first weight [{hidden_dim}, V], got {shape}")
        return True
    if weight.ndim != 2:
        raise ValueError(f"lm_head must be a matrix, got shape {shape}")
    if shape[1] == hidden_dim:
        return False
    if shape[0] == hidden_dim:
        return True
    raise ValueError(
        f"Could not infer lm_head layout from hidden dim {hidden_dim} and weight shape {shape}"
    )


# ------------------------------------------------------------------ host path --
class _HostTiledLinearCrossEntropy(torch.autograd.Function):
    """Vocabulary-streaming linear CE for host (CPU) tensors.

    Counterpart of the reference's ``_TiledLinearCrossEntropy``
    (tiled_linear_cross_entropy.py:56-277).  The running log-sum-exp is carried
    as one number per row and merged tile by tile with ``logaddexp``; backward
    re-forms each logits tile and accumulates the three gradients in float32.
    """

    @staticmethod
    def _tile_logits(ctx_like, h, weight, bias, lo, hi):
        w = weight[:, lo:hi] if ctx_like.weight_dim_first else weight[lo:hi]
        w = w.to(ctx_like.compute_dtype)
        raw = (h @ w) if ctx_like.weight_dim_first else (h @ w.t())
        raw = raw.to(torch.float32)
        if bias is not None:
            raw = raw + bias[lo:hi].to(torch.float32)
        if ctx_like.logit_softcap > 0:
            squashed = torch.tanh(raw / ctx_like.logit_softcap)
            logits = squashed * ctx_like.logit_softcap
        else:
            squashed = None
            logits = raw
        if lo <= ctx_like.exclude_index < hi:
            logits = logits.clone()
            logits[:, ctx_like.exclude_index - lo] = -float("inf")
        return logits, squashed

    @staticmethod
    def forward(  # type: ignore[override]
        ctx,
        hidden: torch.Tensor,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor],
        labels: torch.Tensor,
        row_block_size: int,
        vocab_block_size: int,
        reduction: str,
        ignore_index: int,
        exclude_index: int,
        compute_dtype: torch.dtype,
        weight_dim_first: bool,
        logit_softcap: float,
    ):
        if hidden.ndim not in {2, 3}:
            raise ValueError(f"hidden must be [N, D] or [B, S, D], got {hidden.shape}")
        if labels.shape != hidden.shape[:-1]:
            raise ValueError(
                f"labels shape {tuple(labels.shape)} must match hidden prefix "
                f"{tuple(hidden.shape[:-1])}"
            )
        if reduction not in {"mean", "sum", "none"}:
            raise ValueError("reduction must be 'mean', 'sum', or 'none'")
        if row_block_size <= 0 or vocab_block_size <= 0:
            raise ValueError("row_block_size and vocab_block_size must be positive")

        rows = hidden.reshape(-1, hidden.shape[-1])
        targets = labels.reshape(-1).to(torch.long)
        n = rows.shape[0]
        vocab = weight.shape[1] if weight_dim_first else weight.shape[0]
        if bias is not None and tuple(bias.shape) != (vocab,):
            raise ValueError(f"bias must have shape ({vocab},), got {tuple(bias.shape)}")

        keep = targets != ignore_index
        kept = targets[keep]
        if kept.numel():
            if int(kept.min()) < 0 or int(kept.max()) >= vocab:
                raise ValueError(
                    f"labels must be in [0, {vocab}) or ignore_index={ignore_index}"
                )
            if exclude_index >= 0 and bool((kept == exclude_index).any()):
                raise ValueError("labels may not equal exclude_index")

        ctx.compute_dtype = compute_dtype
        ctx.weight_dim_first = weight_dim_first
        ctx.exclude_index = exclude_index
        ctx.logit_softcap = float(logit_softcap)

        lse = torch.full((n,), -float("inf"), dtype=torch.float32, device=rows.device)
        picked = torch.zeros(n, dtype=torch.float32, device=rows.device)
        safe_targets = torch.where(keep, targets, torch.zeros_like(targets))
        for r0 in range(0, n, row_block_size):
            r1 = min(r0 + row_block_size, n)
            h = rows[r0:r1].to(compute_dtype)
            for lo in range(0, vocab, vocab_block_size):
                hi = min(lo + vocab_block_size, vocab)
                logits, _ = _HostTiledLinearCrossEntropy._tile_logits(
                    ctx, h, weight, bias, lo, hi
                )
                lse[r0:r1] = torch.logaddexp(lse[r0:r1], torch.logsumexp(logits, dim=-1))
                y = safe_targets[r0:r1]
                here = keep[r0:r1] & (y >= lo) & (y < hi)
                local = (y - lo).clamp(0, hi - lo - 1)
                picked[r0:r1] += torch.where(
                    here, logits.gather(1, local[:, None]).squeeze(1), torch.zeros_like(lse[r0:r1])
                )
        losses = torch.where(keep, lse - picked, torch.zeros_like(lse))
        valid_count = keep.sum().to(torch.float32)

        ctx.save_for_backward(rows, weight, bias, targets, lse, keep)
        ctx.hidden_shape = hidden.shape
        ctx.row_block_size = row_block_size
        ctx.vocab_block_size = vocab_block_size
        ctx.reduction = reduction
        ctx.vocab = vocab
        ctx.valid_count = valid_count
        if reduction == "none":
            return losses.reshape(labels.shape)
        if reduction == "sum":
            return losses.sum()
        return losses.sum() / valid_count

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        rows, weight, bias, targets, lse, keep = ctx.saved_tensors
        n = rows.shape[0]
        if ctx.reduction == "none":
            scale = grad_output.reshape(-1).to(torch.float32)
        elif ctx.reduction == "sum":
            scale = grad_output.to(torch.float32).expand(n)
        else:
            scale = (grad_output.to(torch.float32) / ctx.valid_count).expand(n)
        scale = torch.where(keep, scale, torch.zeros_like(scale))

        grad_rows = torch.zeros(rows.shape, dtype=torch.float32, device=rows.device)
        grad_weight = torch.zeros(weight.shape, dtype=torch.float32, device=weight.device)
        grad_bias = None if bias is None else torch.zeros(bias.shape, dtype=torch.float32)
        for r0 in range(0, n, ctx.row_block_size):
            r1 = min(r0 + ctx.row_block_size, n)
            h = rows[r0:r1].to(ctx.compute_dtype)
            h32 = rows[r0:r1].to(torch.float32)
            y = targets[r0:r1]
            for lo in range(0, ctx.vocab, ctx.vocab_block_size):
                hi = min(lo + ctx.vocab_block_size, ctx.vocab)
                logits, squashed = _HostTiledLinearCrossEntropy._tile_logits(
                    ctx, h, weight, bias, lo, hi
                )
                g = torch.exp(logits - lse[r0:r1, None])          # softmax tile (0 at excluded)
                here = keep[r0:r1] & (y >= lo) & (y < hi)
                hit = torch.nonzero(here).flatten()
                g[hit, y[hit] - lo] -= 1.0
                g = g * scale[r0:r1, None]
                if squashed is not None:
                    g = g * (1.0 - squashed * squashed)
                if ctx.weight_dim_first:
                    w32 = weight[:, lo:hi].to(torch.float32)
                    grad_rows[r0:r1] += g @ w32.t()
                    grad_weight[:, lo:hi] += h32.t() @ g
                else:
                    w32 = weight[lo:hi].to(torch.float32)
                    grad_rows[r0:r1] += g @ w32
                    grad_weight[lo:hi] += g.t() @ h32
                if grad_bias is not None:
                    grad_bias[lo:hi] += g.sum(dim=0)
        grad_hidden = grad_rows.reshape(ctx.hidden_shape).to(rows.dtype)
        grad_weight = grad_weight.to(weight.dtype)
        if grad_bias is not None:
            grad_bias = grad_bias.to(bias.dtype)
        return (grad_hidden, grad_weight, grad_bias) + (None,) * 9


# ---------------------------------------------------------------- device path --
def _device_forward(ctx, hidden, weight, bias, labels, reduction, ignore_index, exclude_index,
                    compute_dtype, weight_dim_first, logit_softcap, mode):
    """Shared forward of the trainable- and frozen-head autograd functions.

    Mirrors ``_ChunkedDenseLinearCrossEntropy.forward``
    (tiled_linear_cross_entropy.py:282-331) with the row compaction of the loss
    call sites (nemotron/model.py:4234-4253) folded in.
    """
    from . import chunked_linear_ce_native as native

    hidden_flat = hidden.reshape(-1, hidden.shape[-1]).contiguous()
    labels_flat = labels.reshape(-1).to(torch.long).contiguous()
    n = hidden_flat.shape[0]
    # A [H, V] head is read in place where the library can (16-bit inputs, H and V
    # multiples of 64) and the row count is read back or rows stay in place; otherwise
    # it is re-laid to [V, H] once here and the copy is kept for the backward.
    in_place = mode != "device" and native.dim_first_in_place(weight, weight_dim_first)
    if in_place or not weight_dim_first:
        weight_vf = weight.contiguous()
    else:
        weight_vf = weight.t().contiguous()
    if bias is not None:
        bias = bias.contiguous()

    if in_place and mode == "sync":
        # the entry points that take a device-side row count read a [V, H] head only:
        # compact with the count read back, as the reference's call sites do
        row_idx, m = native.compact_rows(labels_flat, ignore_index)
        row_count = None
        if m == n:
            rows, targets, row_idx = hidden_flat, labels_flat, None
        else:
            rows = native.gather_rows(hidden_flat, row_idx)
            targets = native.gather_rows(labels_flat, row_idx)
    else:
        rows, targets, _, row_idx, row_count, m = native.compact_loss_rows(
            hidden_flat, labels_flat, None, ignore_index, mode)

    # Gradients while the logits exist (3 contractions instead of 4): when some input
    # needs a gradient and the library takes the operands (options.GRADIENT_MODES).
    # grad_hidden is linear in each row's upstream gradient, so it can be formed for
    # any reduction; grad_weight needs the upstream gradient inside its contraction,
    # so with per-token losses (reduction "none") it must be the postponed contraction,
    # which exists when all rows form one block.
    wants_grad = bool(ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
    ctx.fused = (
        wants_grad and options.get_gradient_mode() == "forward"
        and native.fused_gradients_supported(rows, weight_vf, bias, in_place or weight_dim_first)
    )
    can_wait = ctx.fused and bool(ctx.needs_input_grad[1]) and native.weight_grad_can_wait(
        m, rows.shape[1], weight_vf.shape[0], rows.dtype)
    if reduction == "none" and bool(ctx.needs_input_grad[1]) and not can_wait:
        ctx.fused = False
    if ctx.fused:
        # (rows compacted with the count read back carry up to 63 zero rows of padding)
        rows, targets = rows[:m], targets[:m]
        # all rows in one block: the grad_weight contraction waits for the upstream
        # gradient and is stored in the input dtype at once (no float32 [V, H] buffer)
        ctx.postponed = can_wait
        losses, lse, valid_count, grad_rows32, grad_weight32 = native.forward_with_gradients(
            rows, weight_vf, targets, ignore_index=ignore_index, exclude_index=exclude_index,
            logit_softcap=float(logit_softcap),
            compute_weight_grad=bool(ctx.needs_input_grad[1]), row_idx=row_idx, n_out=n,
            row_count=row_count if mode == "device" else None,
            postpone_weight_grad=ctx.postponed,
        )
        ctx.save_for_backward(grad_rows32, grad_weight32, valid_count, row_idx,
                              row_count if mode == "device" else None,
                              rows if ctx.postponed else None)
        ctx.panel_bytes = native.get_panel_bytes()
        ctx.hidden_shape = hidden.shape
        ctx.n_rows, ctx.m = n, m
        ctx.reduction = reduction
        ctx.grad_dtype = hidden.dtype
        ctx.vocab = weight_vf.shape[0]
        if reduction == "none":
            return losses.reshape(labels.shape)
        if reduction == "sum":
            return losses.sum()
        return losses.sum() / valid_count.squeeze(0)
    if row_count is None:
        losses, lse, valid_count = native.forward(
            rows, weight_vf, bias, targets,
            row_block_size=0, ignore_index=ignore_index, exclude_index=exclude_index,
            logit_softcap=float(logit_softcap), compute_dtype=compute_dtype,
            weight_dim_first=in_place, row_idx=row_idx, n_out=n,
        )
    else:
        losses, lse, valid_count, _ = native.masked_loss_forward(
            rows, weight_vf, bias, targets, None, m=m, row_idx=row_idx, row_count=row_count,
            n_out=n, ignore_index=ignore_index, exclude_index=exclude_index,
            logit_softcap=float(logit_softcap), want_losses=True, want_sum=False,
        )
    ctx.save_for_backward(rows, weight_vf, bias, targets, lse, valid_count, row_idx, row_count)
    ctx.hidden_shape = hidden.shape
    ctx.n_rows, ctx.m = n, m
    ctx.reduction = reduction
    ctx.ignore_index = int(ignore_index)
    ctx.exclude_index = int(exclude_index)
    ctx.compute_dtype = compute_dtype
    ctx.weight_dim_first = weight_dim_first
    ctx.in_place = in_place
    ctx.logit_softcap = float(logit_softcap)
    # the backward may run on an autograd worker thread, which does not see this
    # thread's context: the panel budget in force now travels with the node
    ctx.panel_bytes = native.get_panel_bytes()
    if reduction == "none":
        return losses.reshape(labels.shape)
    if reduction == "sum":
        return losses.sum()
    return losses.sum() / valid_count.squeeze(0)


def _device_backward(ctx, grad_output, frozen: bool):
    from . import chunked_linear_ce_native as native

    if ctx.fused:
        grad_rows32, grad_weight32, valid_count, row_idx, row_count, rows = ctx.saved_tensors
        grad_hidden, grad_weight = native.apply_grad_output(
            grad_rows32, None if ctx.postponed else grad_weight32, grad_output, valid_count,
            reduction=ctx.reduction, dtype=ctx.grad_dtype, row_idx=row_idx, n_out=ctx.n_rows,
            vocab=ctx.vocab, row_count=row_count,
        )
        if ctx.postponed and not frozen:
            # grad_weight32 is the forward's workspace: its panel still holds every row
            grad_weight = native.grad_weight_from_panel(
                rows, grad_weight32, grad_output, valid_count, reduction=ctx.reduction,
                vocab=ctx.vocab, panel_bytes=ctx.panel_bytes, row_count=row_count,
                row_idx=row_idx, n_out=ctx.n_rows,
            )
        return (grad_hidden.reshape(ctx.hidden_shape), None if frozen else grad_weight,
                None) + (None,) * 9
    rows, weight_vf, bias, targets, lse, valid_count, row_idx, row_count = ctx.saved_tensors
    with native.panel_budget(ctx.panel_bytes):
        if row_count is None:
            call = native.backward_frozen_weight if frozen else native.backward
            grad_hidden, grad_weight, grad_bias = call(
                rows, weight_vf, bias, targets, lse, valid_count, grad_output,
                row_block_size=0, reduction=ctx.reduction, ignore_index=ctx.ignore_index,
                exclude_index=ctx.exclude_index, logit_softcap=ctx.logit_softcap,
                compute_dtype=ctx.compute_dtype, weight_dim_first=ctx.in_place,
                row_idx=row_idx, n_out=ctx.n_rows,
            )
        else:
            grad_hidden, grad_weight, grad_bias = native.masked_loss_backward(
                rows, weight_vf, bias, targets, None, lse, valid_count, grad_output,
                reduction=ctx.reduction, m=ctx.m, row_idx=row_idx, row_count=row_count,
                n_out=ctx.n_rows, ignore_index=ctx.ignore_index, exclude_index=ctx.exclude_index,
                logit_softcap=ctx.logit_softcap, compute_weight_grad=not frozen,
            )
    if not frozen and ctx.weight_dim_first and not ctx.in_place:
        grad_weight = grad_weight.t().contiguous()
    return (
        grad_hidden.reshape(ctx.hidden_shape),
        None if frozen else grad_weight,
        None if bias is None else grad_bias,
    ) + (None,) * 9


class _ChunkedDenseLinearCrossEntropy(torch.autograd.Function):
    """Device path, trainable head (tiled_linear_cross_entropy.py:280-368)."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels, row_block_size, reduction, ignore_index,
                exclude_index, compute_dtype, weight_dim_first, logit_softcap,
                compaction="sync"):  # type: ignore[override]
        del row_block_size
        return _device_forward(ctx, hidden, weight, bias, labels, reduction, ignore_index,
                               exclude_index, compute_dtype, weight_dim_first, logit_softcap,
                               compaction)

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        return _device_backward(ctx, grad_output, frozen=False)


class _ChunkedFrozenLinearCrossEntropy(torch.autograd.Function):
    """Device path, frozen head: no weight gradient
    (tiled_linear_cross_entropy.py:371-435)."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels, row_block_size, reduction, ignore_index,
                exclude_index, compute_dtype, weight_dim_first, logit_softcap,
                compaction="sync"):  # type: ignore[override]
        del row_block_size
        return _device_forward(ctx, hidden, weight, bias, labels, reduction, ignore_index,
                               exclude_index, compute_dtype, weight_dim_first, logit_softcap,
                               compaction)

    @staticmethod
    def backward(ctx, grad_output):  # type: ignore[override]
        return _device_backward(ctx, grad_output, frozen=True)


def _should_use_chunked_dense_ce(hidden, weight, bias, labels, compute_dtype) -> bool:
    # same admission rule as tiled_linear_cross_entropy.py:438-456
    if not (hidden.is_cuda and weight.is_cuda and labels.is_cuda):
        return False
    floats = {torch.float16, torch.bfloat16, torch.float32}
    if hidden.dtype not in floats or weight.dtype != hidden.dtype:
        return False
    if bias is not None and bias.dtype != hidden.dtype:
        return False
    return compute_dtype in floats


def tiled_linear_cross_entropy(
    hidden: torch.Tensor,
    lm_head: torch.Tensor,
    labels: torch.Tensor,
    *,
    bias: Optional[torch.Tensor] = None,
    vocab_block_size: int = 0,
    reduction: str = "mean",
    ignore_index: int = -100,
    exclude_index: Optional[int] = None,
    logit_softcap: float | None = None,
    dtype: torch.dtype | str = torch.float32,
    weight_layout: str = "auto",
    compaction: Optional[str] = None,
) -> torch.Tensor:
    """Linear projection plus cross entropy without materializing [N, V] logits.

    Args:
      hidden: token representations, [B, S, D] or [N, D].
      lm_head: output projection, [V, D] ("vocab_first") or [D, V] ("dim_first");
        "auto" infers the layout and needs an explicit choice for square heads.
      labels: target ids, [B, S] or [N]; ``ignore_index`` rows carry no loss.
      bias: optional [V] output bias.
      vocab_block_size: vocabulary entries per tile of the host path (0 = all);
        the device path tiles by its own plan.
      reduction: "mean" (over non-ignored rows), "sum" or "none".
      exclude_index: vocabulary id removed from the softmax (e.g. the mask token).
      logit_softcap: positive cap applied as ``cap * tanh(logit / cap)``.
      dtype: matmul dtype of the host path; accumulation is float32 everywhere.
      compaction: how the device path removes ignored rows ("sync", "device" or
        "none", see ``options.COMPACTION_MODES``); None takes the mode of the
        calling context (``compaction_mode(...)``).  Not part of the reference's
        signature; the host path ignores it.

    Returns the same value as ``F.cross_entropy(hidden @ lm_head.T + bias, labels)``
    up to floating-point associativity; float32, shaped like ``labels`` for
    reduction "none", scalar otherwise.
    """
    if hidden.shape[:-1] != labels.shape:
        raise ValueError(
            f"labels shape {tuple(labels.shape)} must match hidden prefix "
            f"{tuple(hidden.shape[:-1])}"
        )
    compute_dtype = _canonical_dtype(dtype)
    weight_dim_first = _infer_weight_layout(hidden.shape[-1], lm_head, weight_layout)
    excluded = -1 if exclude_index is None else int(exclude_index)
    softcap = 0.0 if logit_softcap is None else float(logit_softcap)
    if _should_use_chunked_dense_ce(hidden, lm_head, bias, labels, compute_dtype):
        if reduction not in {"mean", "sum", "none"}:
            raise ValueError("reduction must be 'mean', 'sum', or 'none'")
        implementation = (
            _ChunkedDenseLinearCrossEntropy
            if lm_head.requires_grad
            else _ChunkedFrozenLinearCrossEntropy
        )
        return implementation.apply(
            hidden, lm_head, bias, labels, 0, reduction, int(ignore_index), excluded,
            compute_dtype, weight_dim_first, softcap, resolve_compaction(compaction),
        )
    if hidden.is_cuda or lm_head.is_cuda or labels.is_cuda:
        raise RuntimeError(
            "device tiled_linear_cross_entropy requires hidden, lm_head, bias and labels "
            "on the GPU with one floating dtype; refusing to fall back to the host "
            "tiled implementation."
        )
    n_rows = hidden.reshape(-1, hidden.shape[-1]).shape[0]
    vocab = lm_head.shape[1] if weight_dim_first else lm_head.shape[0]
    tile = int(vocab) if vocab_block_size <= 0 else int(vocab_block_size)
    return _HostTiledLinearCrossEntropy.apply(
        hidden, lm_head, bias, labels, int(max(n_rows, 1)), tile, reduction,
        int(ignore_index), excluded, compute_dtype, weight_dim_first, softcap,
    )
