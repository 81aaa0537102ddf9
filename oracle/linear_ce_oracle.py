"""CPU oracle for the fused linear cross-entropy path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module: it is the checker for
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``.  It restates, on the CPU, what the reference computes for this
path; the reference is Python/CUDA and is read, not run.

What each function follows in the reference (paths relative to its tree):

  dense_linear_ce          the unfused path matmul -> (+bias) -> tanh soft cap ->
                           excluded column -> log-softmax -> masked NLL, with the
                           op order of ce_forward_kernel
                           (dllm_parallel/core/csrc/fused_linear_ce/fused_linear_ce_cuda.cu:156-224)
                           and the reductions of
                           dllm_parallel/core/kernels/tiled_linear_cross_entropy.py:327-331.
  dense_linear_ce_grads    ce_grad_logits_kernel + the two gradient GEMMs
                           (fused_linear_ce_cuda.cu:226-290, :1049-1170); with
                           round_grad_logits=True the logit gradient is rounded to
                           the input dtype before the contractions, as the native
                           path does (:1110-1123).
  online_tiled_linear_ce   the streaming (max, sum) algorithm of the reference's
                           CPU path (tiled_linear_cross_entropy.py:105-149).
  compact_rows             nonzero(labels != ignore) of _compact_valid_loss_rows
                           (dllm_parallel/core/models/backbones/nemotron/model.py:4234-4253).
  vocab_shard_stats        vocab_parallel_ce_stats_kernel (fused_linear_ce_cuda.cu:292-365):
                           per-row (max, sum exp, target logit) of one vocabulary shard.
  dense_soft_embedding     softmax(cap(h W^T)) W * scale, the value that
                           dllm_parallel/core/kernels/streaming_soft_embedding.py:60-148 streams.
  dense_frozen_kl(_grad)   per-token KL(teacher || draft) of two heads and its
                           gradient for the draft hidden states
                           (dflash_kl_forward_kernel / dflash_kl_grad_logits_kernel,
                           fused_linear_ce_cuda.cu:367-480; dense form in
                           dllm_parallel/core/kernels/dflash_kl.py:108-121).
  dense_ce_topk(_grad)     frozen-head CE with the label's probability and the exact
                           top-k logits, and its gradient for hidden
                           (dllm_parallel/core/kernels/dflash_linear_topk.py:100-225).
  masked_token_loss(_grads) the loss method around the operator: hidden * output_multiplier,
                           per-token CE * loss weights, / valid_token_count * loss scale
                           (distributed_block_diffusion_loss,
                           dllm_parallel/core/models/backbones/nemotron/model.py:2084-2151).
  dflash_token_loss(_grads) the DFlash loss method: nonzero(supervised_mask), index_select
                           of hidden / targets / position weights, per-token loss
                           (cross entropy for "paper_ce", KL(teacher || draft) for
                           "speculators_kl"), per-sample numerators by scatter-add,
                           / (normalization_count + 1e-5), mean over samples, * scale
                           (distributed_dflash_loss,
                           dllm_parallel/core/models/backbones/dflash/model.py:862-960).
  segment_weighted_sum     the scatter-add of that method on its own
                           (dflash/model.py:918-937), by a Python loop.
  combine_vocab_shards     the MAX / SUM reductions over shards and the loss of
                           dllm_parallel/core/parallel/tensor_parallel/cross_entropy.py:238-252.

Pinning (tests/test_oracle_pins.py): every function above is checked against
library routines it does not call (torch.nn.functional.cross_entropy, torch
autograd through it, torch.nonzero), against brute-force Python loops on tiny
inputs, against closed forms (uniform logits -> log V, gradient rows summing
to zero, saturated soft cap), against the committed fixtures under
tests/golden/, and against the seeded cases of the reference's own test file
(tests/unit/kernels/test_tiled_linear_cross_entropy.py:61-453), which hold no
stored vectors and compare to the same library routines.  The two shard
functions are pinned by the identity that the statistics of any split of the
vocabulary combine to the dense lse / loss of the unsplit head, by brute force
on a tiny case, and by the special values of the excluded column.  The DFlash
loss method is pinned against the sequence of library calls the reference's
method makes (torch.nonzero, index_select, F.cross_entropy / F.kl_div,
scatter_add_) with autograd through it, and against a per-sample Python loop.
No function here is "parity unpinned".
"""

from __future__ import annotations

from typing import Optional

import numpy as np
import torch


def _logits(hidden, weight, bias, *, weight_dim_first, logit_softcap, exclude_index, dtype):
    h = hidden.reshape(-1, hidden.shape[-1]).to(dtype)
    w = weight.to(dtype)
    raw = h @ (w if weight_dim_first else w.t())
    if bias is not None:
        raw = raw + bias.to(dtype)
    if logit_softcap and logit_softcap > 0:
        squashed = torch.tanh(raw / logit_softcap)
        capped = squashed * logit_softcap
    else:
        squashed = None
        capped = raw
    if exclude_index is not None and exclude_index >= 0:
        capped = capped.clone()
        capped[:, exclude_index] = -float("inf")
    return capped, squashed


def dense_linear_ce(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    bias: Optional[torch.Tensor] = None,
    reduction: str = "mean",
    ignore_index: int = -100,
    exclude_index: Optional[int] = None,
    logit_softcap: Optional[float] = None,
    weight_dim_first: bool = False,
    dtype: torch.dtype = torch.float64,
    return_lse: bool = False,
):
    """Unfused reference value of the loss (and optionally the per-row lse)."""
    logits, _ = _logits(hidden, weight, bias, weight_dim_first=weight_dim_first,
                        logit_softcap=logit_softcap, exclude_index=exclude_index, dtype=dtype)
    y = labels.reshape(-1).to(torch.long)
    keep = y != ignore_index
    row_max = logits.max(dim=-1).values
    lse = row_max + torch.log(torch.exp(logits - row_max[:, None]).sum(dim=-1))
    safe = torch.where(keep, y, torch.zeros_like(y))
    target = logits.gather(1, safe[:, None]).squeeze(1)
    losses = torch.where(keep, lse - target, torch.zeros_like(lse))
    if reduction == "none":
        out = losses.reshape(labels.shape)
    elif reduction == "sum":
        out = losses.sum()
    elif reduction == "mean":
        out = losses.sum() / keep.sum().to(dtype)
    else:
        raise ValueError(reduction)
    return (out, lse) if return_lse else out


def dense_linear_ce_grads(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    grad_output: Optional[torch.Tensor] = None,
    *,
    bias: Optional[torch.Tensor] = None,
    reduction: str = "mean",
    ignore_index: int = -100,
    exclude_index: Optional[int] = None,
    logit_softcap: Optional[float] = None,
    weight_dim_first: bool = False,
    dtype: torch.dtype = torch.float64,
    round_grad_logits: Optional[torch.dtype] = None,
):
    """Analytic (grad_hidden, grad_weight, grad_bias) of ``dense_linear_ce``.

    grad_output follows autograd: shaped like labels for reduction "none",
    scalar otherwise (defaults to ones).
    """
    logits, squashed = _logits(hidden, weight, bias, weight_dim_first=weight_dim_first,
                               logit_softcap=logit_softcap, exclude_index=exclude_index,
                               dtype=dtype)
    y = labels.reshape(-1).to(torch.long)
    n = y.numel()
    keep = y != ignore_index
    lse = torch.logsumexp(logits, dim=-1)
    if grad_output is None:
        grad_output = torch.ones(labels.shape if reduction == "none" else (), dtype=dtype)
    go = grad_output.to(dtype)
    if reduction == "none":
        scale = go.reshape(-1)
    elif reduction == "sum":
        scale = go.reshape(()).expand(n)
    else:
        scale = (go.reshape(()) / keep.sum().to(dtype)).expand(n)
    scale = torch.where(keep, scale, torch.zeros_like(scale))
    g = torch.exp(logits - lse[:, None])
    rows = torch.nonzero(keep).flatten()
    g[rows, y[rows]] -= 1.0
    g = g * scale[:, None]
    if exclude_index is not None and exclude_index >= 0:
        # the excluded column gets no gradient even on a row whose label it is
        # (ce_grad_logits_kernel skips it before the onehot, fused_linear_ce_cuda.cu:270-283)
        g[:, exclude_index] = 0.0
    if squashed is not None:
        g = g * (1.0 - squashed * squashed)
    if round_grad_logits is not None:
        g = g.to(round_grad_logits).to(dtype)
    h = hidden.reshape(-1, hidden.shape[-1]).to(dtype)
    w = weight.to(dtype)
    if weight_dim_first:
        grad_hidden = g @ w.t()
        grad_weight = h.t() @ g
    else:
        grad_hidden = g @ w
        grad_weight = g.t() @ h
    grad_bias = g.sum(dim=0) if bias is not None else None
    return grad_hidden.reshape(hidden.shape), grad_weight, grad_bias


def online_tiled_linear_ce(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    vocab_block_size: int,
    bias: Optional[torch.Tensor] = None,
    ignore_index: int = -100,
    exclude_index: Optional[int] = None,
    logit_softcap: Optional[float] = None,
    dtype: torch.dtype = torch.float32,
):
    """Per-row (losses, lse) by streaming vocabulary tiles with a running
    (max, sum-of-exponentials) pair -- the algorithm every fused kernel of this
    path implements.  Exclusion is applied after the soft cap (true removal)."""
    h = hidden.reshape(-1, hidden.shape[-1]).to(dtype)
    y = labels.reshape(-1).to(torch.long)
    keep = y != ignore_index
    n, vocab = h.shape[0], weight.shape[0]
    run_max = torch.full((n,), -float("inf"), dtype=dtype)
    run_sum = torch.zeros(n, dtype=dtype)
    target = torch.zeros(n, dtype=dtype)
    for lo in range(0, vocab, vocab_block_size):
        hi = min(lo + vocab_block_size, vocab)
        z = h @ weight[lo:hi].to(dtype).t()
        if bias is not None:
            z = z + bias[lo:hi].to(dtype)
        if logit_softcap and logit_softcap > 0:
            z = torch.tanh(z / logit_softcap) * logit_softcap
        if exclude_index is not None and lo <= exclude_index < hi:
            z[:, exclude_index - lo] = -float("inf")
        new_max = torch.maximum(run_max, z.max(dim=-1).values)
        finite = new_max > -float("inf")
        shift = torch.where(finite, new_max, torch.zeros_like(new_max))
        run_sum = torch.where(
            finite,
            run_sum * torch.exp(run_max - shift) + torch.exp(z - shift[:, None]).sum(dim=-1),
            run_sum,
        )
        run_max = new_max
        here = keep & (y >= lo) & (y < hi)
        idx = torch.nonzero(here).flatten()
        target[idx] = z[idx, y[idx] - lo]
    lse = run_max + torch.log(run_sum)
    return torch.where(keep, lse - target, torch.zeros_like(lse)), lse


def compact_rows(labels, ignore_index: int = -100) -> np.ndarray:
    """Ascending int64 indices of labels != ignore_index (numpy)."""
    flat = np.asarray(labels).reshape(-1)
    return np.flatnonzero(flat != ignore_index).astype(np.int64)


def compact_rows_loop(labels, ignore_index: int = -100) -> list[int]:
    """The same by a plain Python loop (tiny inputs only)."""
    return [i for i, y in enumerate(np.asarray(labels).reshape(-1).tolist()) if y != ignore_index]


def relative_max_error(actual: torch.Tensor, expected: torch.Tensor) -> float:
    """max|a - e| / max|e|: the "relative max-norm error" of the gradient bars."""
    a = actual.detach().to(torch.float64).cpu()
    e = expected.detach().to(torch.float64).cpu()
    denom = float(e.abs().max())
    if denom == 0.0:
        return float(a.abs().max())
    return float((a - e).abs().max()) / denom


def vocab_shard_stats(
    hidden: torch.Tensor,
    weight_shard: torch.Tensor,
    labels: torch.Tensor,
    *,
    vocab_start: int,
    bias: Optional[torch.Tensor] = None,
    ignore_index: int = -100,
    exclude_index: int = -1,
    logit_softcap: float = 0.0,
    dtype: torch.dtype = torch.float64,
):
    """(local_max, local_sum, target_logits, valid_count) of the weight rows
    [vocab_start, vocab_start + V_local); labels and exclude_index are global ids."""
    h = hidden.reshape(-1, hidden.shape[-1]).to(dtype)
    z = h @ weight_shard.to(dtype).t()
    if bias is not None:
        z = z + bias.to(dtype)
    if logit_softcap and logit_softcap > 0:
        z = torch.tanh(z / logit_softcap) * logit_softcap
    v_local = weight_shard.shape[0]
    y = labels.reshape(-1).to(torch.long)
    valid = y != ignore_index
    local_exclude = exclude_index - vocab_start
    masked = z.clone()
    if 0 <= local_exclude < v_local:
        masked[:, local_exclude] = -float("inf")
    local_max = masked.max(dim=1).values
    shifted = masked - torch.where(torch.isinf(local_max), torch.zeros_like(local_max),
                                   local_max)[:, None]
    local_sum = torch.exp(shifted).sum(dim=1)
    local_sum = torch.where(torch.isinf(local_max), torch.zeros_like(local_sum), local_sum)
    y_local = y - vocab_start
    here = valid & (y_local >= 0) & (y_local < v_local)
    picked = z.gather(1, y_local.clamp(0, v_local - 1)[:, None])[:, 0]
    target = torch.where(here, picked, torch.zeros_like(picked))
    target = torch.where(here & (y == exclude_index),
                         torch.full_like(target, -float("inf")), target)
    valid_count = valid.sum().to(dtype).reshape(1)
    return local_max, local_sum, target, valid_count


def combine_vocab_shards(stats, labels: torch.Tensor, *, ignore_index: int = -100):
    """Global (losses, lse) from the per-shard statistics: MAX over the maxima,
    SUM of the rescaled sums and of the target logits (every label lives in
    exactly one shard), loss = lse - target on rows that are not ignored."""
    global_max = torch.stack([s[0] for s in stats]).max(dim=0).values
    global_sum = sum(s[1] * torch.exp(s[0] - global_max) for s in stats)
    target = sum(s[2] for s in stats)
    lse = global_max + torch.log(global_sum)
    valid = labels.reshape(-1) != ignore_index
    losses = torch.where(valid, lse - target, torch.zeros_like(lse))
    return losses, lse


def dense_soft_embedding(hidden, weight, *, logit_softcap=None, embedding_scale=1.0,
                         dtype=torch.float64):
    """embedding_scale * softmax(cap(hidden @ weight.T)) @ weight, shaped like hidden."""
    z = hidden.reshape(-1, hidden.shape[-1]).to(dtype) @ weight.to(dtype).t()
    if logit_softcap:
        z = logit_softcap * torch.tanh(z / logit_softcap)
    z = z - z.max(dim=-1, keepdim=True).values
    e = torch.exp(z)
    p = e / e.sum(dim=-1, keepdim=True)
    return (embedding_scale * (p @ weight.to(dtype))).reshape(hidden.shape)


def _kl_parts(draft_hidden, draft_weight, teacher_hidden, teacher_weight, logit_softcap, dtype):
    zd = draft_hidden.to(dtype) @ draft_weight.to(dtype).t()
    zt = teacher_hidden.to(dtype) @ teacher_weight.to(dtype).t()
    dcap = torch.ones_like(zd)
    if logit_softcap:
        td = torch.tanh(zd / logit_softcap)
        dcap = 1.0 - td * td
        zd = logit_softcap * td
        zt = logit_softcap * torch.tanh(zt / logit_softcap)
    log_q = zd - torch.logsumexp(zd, dim=-1, keepdim=True)
    log_p = zt - torch.logsumexp(zt, dim=-1, keepdim=True)
    return log_q, log_p, dcap


def dense_frozen_kl(draft_hidden, draft_weight, teacher_hidden, teacher_weight, *,
                    logit_softcap=None, dtype=torch.float64):
    """losses[r] = sum_v p_t (log p_t - log p_d)."""
    log_q, log_p, _ = _kl_parts(draft_hidden, draft_weight, teacher_hidden, teacher_weight,
                                logit_softcap, dtype)
    return (torch.exp(log_p) * (log_p - log_q)).sum(dim=-1)


def dense_frozen_kl_grad(draft_hidden, draft_weight, teacher_hidden, teacher_weight, grad_output,
                         *, logit_softcap=None, dtype=torch.float64):
    """d sum_r(grad_output[r] * losses[r]) / d draft_hidden
    = ((p_d - p_t) * grad_output[r] * cap'(z_d)) @ draft_weight."""
    log_q, log_p, dcap = _kl_parts(draft_hidden, draft_weight, teacher_hidden, teacher_weight,
                                   logit_softcap, dtype)
    g = (torch.exp(log_q) - torch.exp(log_p)) * grad_output.to(dtype)[:, None] * dcap
    return g @ draft_weight.to(dtype)


def _topk_logits(hidden, weight, output_multiplier, logit_softcap, dtype):
    raw = hidden.to(dtype) @ weight.to(dtype).t() * output_multiplier
    if logit_softcap:
        th = torch.tanh(raw / logit_softcap)
        return logit_softcap * th, output_multiplier * (1.0 - th * th)
    return raw, torch.full_like(raw, output_multiplier)


def dense_ce_topk(hidden, weight, labels, top_k, *, output_multiplier=1.0, logit_softcap=None,
                  dtype=torch.float64):
    """(loss, probability, top_values, top_ids, lse); the top-k sorted descending,
    equal values in ascending id order."""
    z, _ = _topk_logits(hidden, weight, output_multiplier, logit_softcap, dtype)
    lse = torch.logsumexp(z, dim=-1)
    loss = lse - z.gather(1, labels.reshape(-1, 1).to(torch.long))[:, 0]
    order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top_k]
    return loss, torch.exp(-loss), z.gather(1, order), order, lse


def dense_ce_topk_grad(hidden, weight, labels, top_ids, grad_loss, grad_probability,
                       grad_top_values, *, output_multiplier=1.0, logit_softcap=None,
                       dtype=torch.float64):
    """d(sum grad_loss*loss + grad_probability*probability + grad_top_values*top_values)/d hidden."""
    z, dz = _topk_logits(hidden, weight, output_multiplier, logit_softcap, dtype)
    lse = torch.logsumexp(z, dim=-1)
    y = labels.reshape(-1, 1).to(torch.long)
    prob = torch.exp(z.gather(1, y)[:, 0] - lse)
    ce_scale = grad_loss.to(dtype) - grad_probability.to(dtype) * prob
    g = torch.exp(z - lse[:, None]) * ce_scale[:, None]
    g.scatter_add_(1, y, -ce_scale[:, None])
    if grad_top_values is not None:
        g.scatter_add_(1, top_ids.to(torch.long), grad_top_values.to(dtype))
    return (g * dz) @ weight.to(dtype)


def masked_token_loss(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    loss_weights: torch.Tensor,
    valid_token_count: float,
    *,
    bias: Optional[torch.Tensor] = None,
    exclude_index: Optional[int] = None,
    output_multiplier: Optional[float] = None,
    logit_softcap: Optional[float] = None,
    loss_scale: float = 1.0,
    dtype: torch.dtype = torch.float64,
    round_scaled_hidden: bool = False,
):
    """``sum_r CE_r * w_r / valid_token_count * loss_scale`` over the rows whose
    label is not -100, CE taken on ``hidden * output_multiplier``
    (nemotron/model.py:2084-2086, :2099-2151).  The multiplication is done in
    ``dtype``; with ``round_scaled_hidden`` the product is first rounded to the
    dtype of ``hidden``, which is where the reference rounds it
    (``compact_hidden * float(multiplier)`` on the 16-bit tensor)."""
    h = hidden.reshape(-1, hidden.shape[-1])
    if output_multiplier is not None and round_scaled_hidden:
        h = (h * float(output_multiplier)).to(hidden.dtype).to(dtype)
    else:
        h = h.to(dtype)
        if output_multiplier is not None:
            h = h * float(output_multiplier)
    token_losses = dense_linear_ce(h, weight, labels.reshape(-1), bias=bias, reduction="none",
                                   exclude_index=exclude_index, logit_softcap=logit_softcap,
                                   dtype=dtype)
    w = loss_weights.reshape(-1).to(dtype)
    keep = labels.reshape(-1) != -100
    loss_sum = (token_losses * torch.where(keep, w, torch.zeros_like(w))).sum()
    return loss_sum / valid_token_count * float(loss_scale)


def masked_token_loss_grads(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    loss_weights: torch.Tensor,
    valid_token_count: float,
    *,
    bias: Optional[torch.Tensor] = None,
    exclude_index: Optional[int] = None,
    output_multiplier: Optional[float] = None,
    logit_softcap: Optional[float] = None,
    loss_scale: float = 1.0,
    dtype: torch.dtype = torch.float64,
):
    """Analytic (grad_hidden, grad_weight, grad_bias) of ``masked_token_loss``:
    the per-token scale is ``w_r / valid_token_count * loss_scale``; the chain
    rule through ``hidden * output_multiplier`` multiplies grad_hidden by the
    multiplier while grad_weight sees the multiplied hidden states."""
    mult = 1.0 if output_multiplier is None else float(output_multiplier)
    h = hidden.reshape(-1, hidden.shape[-1]).to(dtype) * mult
    per_token = loss_weights.reshape(-1).to(dtype) / valid_token_count * float(loss_scale)
    grad_scaled, grad_weight, grad_bias = dense_linear_ce_grads(
        h, weight, labels.reshape(-1), per_token, bias=bias, reduction="none",
        exclude_index=exclude_index, logit_softcap=logit_softcap, dtype=dtype)
    return (grad_scaled * mult).reshape(hidden.shape), grad_weight, grad_bias


def segment_weighted_sum(values, weights, row_idx, segment_length: int, n_segments: int):
    """out[s] = sum of values[r] * weights[r] over the rows whose position
    row_idx[r] lies in sample s (float64, plain Python loop)."""
    out = [0.0] * n_segments
    for r in range(len(row_idx)):
        s = int(row_idx[r]) // int(segment_length)
        out[s] += float(values[r]) * (1.0 if weights is None else float(weights[r]))
    return torch.tensor(out, dtype=torch.float64)


def _dflash_rows(hidden_states, supervised_mask, position_weights, dtype):
    keep = supervised_mask.reshape(-1).bool()
    idx = torch.nonzero(keep, as_tuple=False).flatten()
    rows = hidden_states.reshape(-1, hidden_states.shape[-1])[idx]
    weights = position_weights.reshape(-1)[idx].to(dtype)
    return idx, rows, weights


def dflash_token_loss(
    hidden_states: torch.Tensor,
    target_token_ids: torch.Tensor,
    supervised_mask: torch.Tensor,
    position_weights: torch.Tensor,
    draft_weight: torch.Tensor,
    normalization_count: torch.Tensor,
    *,
    loss_kind: str,
    teacher_hidden_states: Optional[torch.Tensor] = None,
    teacher_weight: Optional[torch.Tensor] = None,
    logit_softcap: Optional[float] = None,
    loss_scale: float = 1.0,
    dtype: torch.dtype = torch.float64,
):
    """mean_b( sum_{r in sample b} loss_r * w_r / (normalization_count[b] + 1e-5) ) * loss_scale
    over the supervised positions of a [B, T] batch (dflash/model.py:862-960).
    ``teacher_hidden_states`` are taken as already normalised (the reference
    applies its verifier norm, a module outside this path, just before)."""
    batch, tokens = supervised_mask.shape
    idx, rows, weights = _dflash_rows(hidden_states, supervised_mask, position_weights, dtype)
    if idx.numel() == 0:
        return torch.zeros((), dtype=dtype)
    if loss_kind == "paper_ce":
        labels = target_token_ids.reshape(-1)[idx]
        token_loss = dense_linear_ce(rows, draft_weight, labels, reduction="none",
                                     logit_softcap=logit_softcap, dtype=dtype)
    elif loss_kind == "speculators_kl":
        teacher = teacher_hidden_states.reshape(-1, teacher_hidden_states.shape[-1])[idx]
        token_loss = dense_frozen_kl(rows, draft_weight, teacher, teacher_weight,
                                     logit_softcap=logit_softcap, dtype=dtype)
    else:
        raise ValueError(f"unsupported DFlash loss {loss_kind!r}")
    numerators = torch.zeros(batch, dtype=dtype)
    numerators.scatter_add_(0, idx // tokens, token_loss.to(dtype) * weights)
    return (numerators / (normalization_count.to(dtype) + 1.0e-5)).mean() * float(loss_scale)


def dflash_token_loss_grads(
    hidden_states: torch.Tensor,
    target_token_ids: torch.Tensor,
    supervised_mask: torch.Tensor,
    position_weights: torch.Tensor,
    draft_weight: torch.Tensor,
    normalization_count: torch.Tensor,
    *,
    loss_kind: str,
    teacher_hidden_states: Optional[torch.Tensor] = None,
    teacher_weight: Optional[torch.Tensor] = None,
    logit_softcap: Optional[float] = None,
    loss_scale: float = 1.0,
    dtype: torch.dtype = torch.float64,
):
    """Analytic (grad_hidden_states, grad_draft_weight) of ``dflash_token_loss``
    (grad_draft_weight is None for the KL, whose heads are frozen): the per-token
    scale is w_r / (normalization_count[b_r] + 1e-5) / B * loss_scale."""
    batch, tokens = supervised_mask.shape
    idx, rows, weights = _dflash_rows(hidden_states, supervised_mask, position_weights, dtype)
    grad_hidden = torch.zeros(hidden_states.reshape(-1, hidden_states.shape[-1]).shape, dtype=dtype)
    if idx.numel() == 0:
        return grad_hidden.reshape(hidden_states.shape), None
    per_token = weights / (normalization_count.to(dtype)[idx // tokens] + 1.0e-5) / batch \
        * float(loss_scale)
    if loss_kind == "paper_ce":
        labels = target_token_ids.reshape(-1)[idx]
        grad_rows, grad_weight, _ = dense_linear_ce_grads(
            rows, draft_weight, labels, per_token, reduction="none",
            logit_softcap=logit_softcap, dtype=dtype)
    elif loss_kind == "speculators_kl":
        teacher = teacher_hidden_states.reshape(-1, teacher_hidden_states.shape[-1])[idx]
        grad_rows = dense_frozen_kl_grad(rows, draft_weight, teacher, teacher_weight, per_token,
                                         logit_softcap=logit_softcap, dtype=dtype)
        grad_weight = None
    else:
        raise ValueError(f"unsupported DFlash loss {loss_kind!r}")
    grad_hidden[idx] = grad_rows.to(dtype)
    return grad_hidden.reshape(hidden_states.shape), grad_weight
