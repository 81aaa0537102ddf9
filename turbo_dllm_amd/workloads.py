"""Seeded synthetic workloads for the fused linear cross-entropy path.

Shapes and label/mask distributions of the benchmark configurations (LM-head
sizes of Qwen3-8B and Gemma-style models, block-diffusion masking as produced
by the reference's corruption runtime,
dllm_parallel/core/objectives/runtime.py:153-197: ``labels = where(mask, x0,
-100)`` with a per-sequence or per-block masking rate t ~ U(0, 1)).  Tensors are
generated on the CPU from one ``torch.Generator`` in float32 and then cast, so
host and device consumers see identical bits.  ``scale`` shrinks token and
vocabulary counts for CPU-sized parity cases while keeping the hidden size.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

IGNORE_INDEX = -100


@dataclass
class Workload:
    name: str
    hidden: torch.Tensor          # [N, H]
    weight: torch.Tensor          # [V, H]
    labels: torch.Tensor          # [N] int64, IGNORE_INDEX on rows without loss
    logit_softcap: Optional[float] = None
    seed: int = 0

    @property
    def n_rows(self) -> int:
        return int(self.labels.numel())

    @property
    def n_loss_rows(self) -> int:
        return int((self.labels != IGNORE_INDEX).sum())

    def to(self, device) -> "Workload":
        return Workload(self.name, self.hidden.to(device), self.weight.to(device),
                        self.labels.to(device), self.logit_softcap, self.seed)


def _tensors(gen, n, h, v, dtype, hidden_std=1.0, weight_std=0.02):
    hidden = (torch.randn(n, h, generator=gen) * hidden_std).to(dtype)
    weight = (torch.randn(v, h, generator=gen) * weight_std).to(dtype)
    return hidden, weight


def _uniform_labels(gen, n, v):
    return torch.randint(0, v, (n,), generator=gen, dtype=torch.long)


def _apply_mask(labels, keep):
    return torch.where(keep, labels, torch.full_like(labels, IGNORE_INDEX))


def small_head(seed=0, scale=1, dtype=torch.bfloat16) -> Workload:
    """2048 tokens, H=1024, V=32000, each row loss-bearing with p=0.5."""
    gen = torch.Generator().manual_seed(seed)
    n, h, v = 2048 // scale, 1024, 32000 // scale
    hidden, weight = _tensors(gen, n, h, v, dtype)
    labels = _uniform_labels(gen, n, v)
    keep = torch.rand(n, generator=gen) < 0.5
    return Workload("small_head", hidden, weight, _apply_mask(labels, keep), seed=seed)


def qwen3_8b_head(seed=0, scale=1, dtype=torch.bfloat16, h=4096) -> Workload:
    """4 sequences x 2048 tokens, H=4096, V=151936; per-sequence rate t~U(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    seqs, seq_len, v = 4, 2048 // scale, 151936 // scale
    n = seqs * seq_len
    hidden, weight = _tensors(gen, n, h, v, dtype)
    labels = _uniform_labels(gen, n, v)
    t = torch.rand(seqs, generator=gen)
    keep = (torch.rand(seqs, seq_len, generator=gen) < t[:, None]).reshape(-1)
    return Workload("qwen3_8b_head", hidden, weight, _apply_mask(labels, keep), seed=seed)


def block_diffusion_shard(seed=0, scale=1, dtype=torch.bfloat16, h=4096,
                          all_rows_loss_bearing=False) -> Workload:
    """One 16384-token sequence as clean+noisy halves (N=32768), H=4096,
    V=151936; loss only on the noisy half, masked per 32-token block at a rate
    t_b~U(0,1).  ``all_rows_loss_bearing`` gives the headline case M=N."""
    gen = torch.Generator().manual_seed(seed)
    seq_len, v, block = 16384 // scale, 151936 // scale, 32
    n = 2 * seq_len
    hidden, weight = _tensors(gen, n, h, v, dtype)
    labels = _uniform_labels(gen, n, v)
    name = "block_diffusion_shard"
    if all_rows_loss_bearing:
        return Workload(name + "_all_rows", hidden, weight, labels, seed=seed)
    n_blocks = seq_len // block
    t = torch.rand(n_blocks, generator=gen)
    noisy_keep = (torch.rand(n_blocks, block, generator=gen) < t[:, None]).reshape(-1)
    keep = torch.cat([torch.zeros(seq_len, dtype=torch.bool), noisy_keep])
    return Workload(name, hidden, weight, _apply_mask(labels, keep), seed=seed)


def gemma_softcap_head(seed=0, scale=1, dtype=torch.bfloat16, h=3840) -> Workload:
    """N=16384, H=3840, V=262144, tanh soft cap 30, 50% of rows loss-bearing."""
    gen = torch.Generator().manual_seed(seed)
    n, v = 16384 // scale, 262144 // scale
    hidden, weight = _tensors(gen, n, h, v, dtype)
    labels = _uniform_labels(gen, n, v)
    keep = torch.rand(n, generator=gen) < 0.5
    return Workload("gemma_softcap_head", hidden, weight, _apply_mask(labels, keep),
                    logit_softcap=30.0, seed=seed)


def sparse_drafter_head(seed=0, scale=1, dtype=torch.bfloat16, h=4096) -> Workload:
    """64 packed sequences of length U{64..1024} (N~35k), H=4096, V=151936, 5% of
    rows loss-bearing, labels Zipf(s=1.1) over vocabulary ids."""
    gen = torch.Generator().manual_seed(seed)
    v = 151936 // scale
    lengths = torch.randint(64 // scale if scale <= 64 else 1, 1024 // scale + 1, (64,),
                            generator=gen)
    n = int(lengths.sum())
    hidden, weight = _tensors(gen, n, h, v, dtype)
    ranks = torch.arange(1, v + 1, dtype=torch.float64)
    labels = torch.multinomial(ranks.pow(-1.1), n, replacement=True, generator=gen)
    keep = torch.rand(n, generator=gen) < 0.05
    return Workload("sparse_drafter_head", hidden, weight, _apply_mask(labels, keep), seed=seed)


CONFIGS = {
    "small_head": small_head,
    "qwen3_8b_head": qwen3_8b_head,
    "block_diffusion_shard": block_diffusion_shard,
    "gemma_softcap_head": gemma_softcap_head,
    "sparse_drafter_head": sparse_drafter_head,
}
