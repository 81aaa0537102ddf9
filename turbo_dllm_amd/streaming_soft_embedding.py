"""Vocabulary logits to soft token embeddings, ``softmax(h W^T) W``, without a
logits buffer.

Same functions, keywords and validation as the reference module
(dllm_parallel/core/kernels/streaming_soft_embedding.py:16-148).  On device
tensors the work runs in the HIP library: the fused forward yields the row
log-sum-exps, then bounded panels of probabilities are contracted with the
weight rows.  ``row_chunk_size`` / ``vocab_chunk_size`` only bound the
reference's torch temporaries; they are validated and otherwise unused there.
Host tensors take a plain dense torch path.
Forward-only, as in the reference (its caller detaches the result).
"""

from __future__ import annotations

from collections.abc import Sequence
from typing import Any

import torch
import torch.nn.functional as F


def _validate(hidden, weights, *, row_chunk_size, vocab_chunk_size, logit_softcap) -> int:
    """Argument checks with the reference's messages (streaming_soft_embedding.py:16-47)."""
    if hidden.ndim < 2:
        raise ValueError("hidden must have at least two dimensions")
    if min(int(row_chunk_size), int(vocab_chunk_size)) <= 0:
        raise ValueError("row and vocabulary chunk sizes must be positive")
    if len(weights) == 0:
        raise ValueError("at least one vocabulary weight shard is required")
    width = int(hidden.shape[-1])
    if any(w.ndim != 2 for w in weights):
        raise ValueError("vocabulary weight must be two-dimensional")
    if any(int(w.shape[1]) != width for w in weights):
        raise ValueError("vocabulary weight hidden dimension does not match hidden")
    if any(w.device != hidden.device for w in weights):
        raise ValueError("hidden and vocabulary weights must share a device")
    if sum(int(w.shape[0]) for w in weights) <= 0:
        raise ValueError("vocabulary must contain at least one row")
    if logit_softcap is not None and float(logit_softcap) <= 0.0:
        raise ValueError("logit_softcap must be positive")
    return width


def _host_soft_embedding(flat, weights, *, row_chunk_size, logit_softcap):
    """Host tensors: dense softmax per block of rows in float32; the
    probabilities are rounded to the weight dtype before the second product,
    like the device path."""
    weight = weights[0] if len(weights) == 1 else torch.cat(weights, dim=0)
    pieces = []
    for rows in flat.split(row_chunk_size, dim=0):
        logits = (rows @ weight.t()).float()
        if logit_softcap is not None:
            cap = float(logit_softcap)
            logits = cap * torch.tanh(logits / cap)
        probabilities = torch.softmax(logits, dim=-1).to(weight.dtype)
        pieces.append((probabilities @ weight).to(flat.dtype))
    return torch.cat(pieces, dim=0)


@torch.no_grad()
def streaming_soft_embedding_from_shards(
    hidden: torch.Tensor,
    weights: Sequence[torch.Tensor],
    *,
    row_chunk_size: int,
    vocab_chunk_size: int,
    logit_softcap: float | None = None,
    embedding_scale: float = 1.0,
) -> torch.Tensor:
    """Soft embedding over the concatenation of the vocabulary shards."""
    weights = tuple(weights)
    hidden_size = _validate(hidden, weights, row_chunk_size=row_chunk_size,
                            vocab_chunk_size=vocab_chunk_size, logit_softcap=logit_softcap)
    original_shape = tuple(hidden.shape)
    flat = hidden.reshape(-1, hidden_size)
    if flat.shape[0] == 0:
        return hidden.detach().clone()
    if flat.is_cuda:
        from . import chunked_linear_ce_native as native

        weight = weights[0] if len(weights) == 1 else torch.cat(weights, dim=0)
        output = native.soft_embedding(
            flat, weight.to(flat.dtype),
            logit_softcap=0.0 if logit_softcap is None else float(logit_softcap),
            embedding_scale=float(embedding_scale),
        )
    else:
        output = _host_soft_embedding(flat, weights, row_chunk_size=int(row_chunk_size),
                                      logit_softcap=logit_softcap)
        if float(embedding_scale) != 1.0:
            output.mul_(float(embedding_scale))
    return output.reshape(original_shape).detach()


@torch.no_grad()
def streaming_soft_embedding(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    *,
    row_chunk_size: int,
    vocab_chunk_size: int,
    logit_softcap: float | None = None,
    embedding_scale: float = 1.0,
    tensor_parallel_group: Any | None = None,
    tensor_parallel_size: int = 1,
) -> torch.Tensor:
    """``softmax(hidden @ weight.T) @ weight`` without full logits.  One GPU is
    built: a tensor-parallel size above 1 raises."""
    _validate(hidden, (weight,), row_chunk_size=row_chunk_size,
              vocab_chunk_size=vocab_chunk_size, logit_softcap=logit_softcap)
    if int(tensor_parallel_size) > 1:
        raise RuntimeError(
            "tensor-parallel streaming soft embeddings are not built in this one-GPU library"
        )
    del tensor_parallel_group
    return streaming_soft_embedding_from_shards(
        hidden, (weight,), row_chunk_size=int(row_chunk_size),
        vocab_chunk_size=int(vocab_chunk_size), logit_softcap=logit_softcap,
        embedding_scale=float(embedding_scale),
    )


__all__ = ["streaming_soft_embedding", "streaming_soft_embedding_from_shards"]
