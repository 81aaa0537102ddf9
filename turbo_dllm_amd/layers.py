"""Output head with the reference's ``parallel_cross_entropy`` method.

One-GPU counterpart of ``VocabParallelLinear``
(dllm_parallel/core/parallel/tensor_parallel/layers.py:273-365): with a tensor
parallel size of 1 the method forwards to ``tiled_linear_cross_entropy`` with
``dtype=x.dtype`` and the vocab-first layout.  Vocabulary sharding over several
GPUs is not part of this build and is rejected at construction.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

from .tiled_linear_cross_entropy import tiled_linear_cross_entropy


class VocabParallelLinear(nn.Module):
    def __init__(
        self,
        in_features: int,
        out_features: int,
        *,
        bias: bool = True,
        tensor_parallel_size: int = 1,
        tensor_parallel_rank: int = 0,
        gather_output: bool = True,
    ) -> None:
        super().__init__()
        if int(tensor_parallel_size) != 1 or int(tensor_parallel_rank) != 0:
            raise NotImplementedError(
                "this build runs on one GPU: tensor_parallel_size must be 1"
            )
        self.in_features = int(in_features)
        self.out_features = int(out_features)
        self.tensor_parallel_size = 1
        self.tensor_parallel_rank = 0
        self.vocab_start, self.vocab_stop = 0, self.out_features
        self.local_out_features = self.out_features
        self.gather_output = bool(gather_output)
        self.weight = nn.Parameter(torch.empty(self.out_features, self.in_features))
        self.bias = nn.Parameter(torch.empty(self.out_features)) if bias else None
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            bound = 1.0 / math.sqrt(self.in_features) if self.in_features > 0 else 0.0
            nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight, self.bias)

    def parallel_cross_entropy(
        self,
        x: torch.Tensor,
        labels: torch.Tensor,
        *,
        ignore_index: int = -100,
        exclude_index: int | None = None,
        vocab_block_size: int = 0,
        reduction: str = "none",
        logit_softcap: float | None = None,
    ) -> torch.Tensor:
        return tiled_linear_cross_entropy(
            x,
            self.weight,
            labels,
            bias=self.bias,
            vocab_block_size=int(vocab_block_size),
            reduction=str(reduction),
            ignore_index=int(ignore_index),
            exclude_index=exclude_index,
            logit_softcap=logit_softcap,
            dtype=x.dtype,
            weight_layout="vocab_first",
        )
