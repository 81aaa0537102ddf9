"""Full-size GPU checks at H=4096, V=151936 through properties that do not need
a dense oracle over every row and column.

  * every per-row loss against the float32 oracle computed in row chunks;
  * grad_hidden on sampled rows and grad_weight on sampled vocabulary rows
    against the oracle formula (each depends on one row / one column only);
  * <grad_weight, weight> == <grad_hidden, hidden>: both equal sum(G * logits);
  * columns of grad_weight sum to zero (softmax minus onehot sums to zero per row);
  * doubling grad_output doubles every gradient bit for bit (scaling by a power
    of two commutes with every rounding on the path);
  * rows without loss get loss 0 and an all-zero grad_hidden row.
"""

import numpy as np
import pytest
import torch

import linear_ce_oracle as oracle
from turbo_dllm_amd import workloads
from turbo_dllm_amd.tiled_linear_cross_entropy import tiled_linear_cross_entropy

pytestmark = pytest.mark.gpu


def say(*parts):
    print("[case]", *parts, flush=True)


def run(dev, wl, grad_scale=1.0):
    hidden = wl.hidden.to(dev).requires_grad_(True)
    weight = wl.weight.to(dev).requires_grad_(True)
    losses = tiled_linear_cross_entropy(hidden, weight, wl.labels.to(dev), reduction="none",
                                        logit_softcap=wl.logit_softcap, dtype=hidden.dtype,
                                        weight_layout="vocab_first")
    m = max(wl.n_loss_rows, 1)
    losses.backward(torch.full_like(losses, grad_scale / m))
    torch.cuda.synchronize()
    return losses.detach().cpu(), hidden.grad.cpu(), weight.grad.cpu()


def oracle_lse_in_chunks(wl, rows, chunk=512):
    weight32 = wl.weight.float()
    losses, lses = [], []
    for lo in range(0, rows.numel(), chunk):
        idx = rows[lo:lo + chunk]
        loss, lse = oracle.dense_linear_ce(wl.hidden[idx], weight32, wl.labels[idx],
                                           reduction="none", logit_softcap=wl.logit_softcap,
                                           dtype=torch.float32, return_lse=True)
        losses.append(loss)
        lses.append(lse)
    return torch.cat(losses), torch.cat(lses)


def test_qwen3_8b_head_full_size(gpu_device):
    wl = workloads.qwen3_8b_head(seed=5)
    n, m = wl.n_rows, wl.n_loss_rows
    say("qwen3_8b_head N", n, "M", m)
    losses, dh, dw = run(gpu_device, wl)
    keep = wl.labels != -100
    rows = torch.nonzero(keep).flatten()

    # every loss-bearing row against the oracle; ignored rows exactly zero
    ref_loss, ref_lse = oracle_lse_in_chunks(wl, rows)
    torch.testing.assert_close(losses[rows], ref_loss, rtol=1e-3, atol=1e-4)
    assert torch.count_nonzero(losses[~keep]) == 0
    assert torch.count_nonzero(dh[~keep]) == 0

    # grad_hidden on sampled rows (depends on that row only)
    gen = torch.Generator().manual_seed(1)
    pick = rows[torch.randperm(m, generator=gen)[:32]]
    rdh, _, _ = oracle.dense_linear_ce_grads(
        wl.hidden[pick], wl.weight, wl.labels[pick], torch.full((32,), 1.0 / m),
        reduction="none", logit_softcap=wl.logit_softcap, dtype=torch.float32)
    err = oracle.relative_max_error(dh[pick], rdh)
    say("grad_hidden sampled rows rel max err", f"{err:.2e}")
    assert err <= 2e-2

    # grad_weight on sampled vocabulary rows: dW[v] = sum_r g[r, v] * h_r
    vs = torch.cat([torch.randint(0, wl.weight.shape[0], (24,), generator=gen),
                    wl.labels[rows[:8]]])                       # include rows that are labels
    h32 = wl.hidden[rows].float()
    z = h32 @ wl.weight[vs].float().t()
    g = torch.exp(z - ref_lse[:, None])
    g -= (wl.labels[rows][:, None] == vs[None, :]).float()
    g /= m
    rdw = g.t() @ h32
    err = oracle.relative_max_error(dw[vs], rdw)
    say("grad_weight sampled rows rel max err", f"{err:.2e}")
    assert err <= 2e-2

    # <dW, W> == <dH, H>
    lhs = float((dw.double() * wl.weight.double()).sum())
    rhs = float((dh.double() * wl.hidden.double()).sum())
    say("inner products", lhs, rhs)
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs))

    # columns of grad_weight sum to zero
    col = dw.double().sum(dim=0).abs()
    scale = dw.double().abs().sum(dim=0)
    assert float((col / scale).max()) <= 2e-2


def test_headline_shape_properties(gpu_device):
    wl = workloads.block_diffusion_shard(seed=0, all_rows_loss_bearing=True)
    say("block_diffusion_shard_all_rows N", wl.n_rows)
    losses, dh, dw = run(gpu_device, wl)
    gen = torch.Generator().manual_seed(2)
    pick = torch.randperm(wl.n_rows, generator=gen)[:64]
    ref_loss, _ = oracle_lse_in_chunks(wl, pick)
    torch.testing.assert_close(losses[pick], ref_loss, rtol=1e-3, atol=1e-4)
    assert bool(torch.isfinite(losses).all())
    lhs = float((dw.double() * wl.weight.double()).sum())
    rhs = float((dh.double() * wl.hidden.double()).sum())
    say("inner products", lhs, rhs)
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs))
    col = dw.double().sum(dim=0).abs()
    scale = dw.double().abs().sum(dim=0)
    assert float((col / scale).max()) <= 2e-2
    # linearity in grad_output, bit for bit
    _, dh2, dw2 = run(gpu_device, wl, grad_scale=2.0)
    assert torch.equal(dh2.float(), dh.float() * 2.0)
    assert torch.equal(dw2.float(), dw.float() * 2.0)


def test_block_diffusion_labels_compaction_full_size(gpu_device):
    from turbo_dllm_amd import chunked_linear_ce_native as native

    torch.manual_seed(0)
    gen = torch.Generator().manual_seed(7)
    labels = torch.randint(0, 151936, (32768,), generator=gen)
    t = torch.rand(512, generator=gen)
    keep = torch.cat([torch.zeros(16384, dtype=torch.bool),
                      (torch.rand(512, 32, generator=gen) < t[:, None]).reshape(-1)])
    labels = torch.where(keep, labels, torch.full_like(labels, -100))
    idx, m = native.compact_rows(labels.to(gpu_device), -100)
    assert np.array_equal(idx.cpu().numpy(), oracle.compact_rows(labels.numpy()))
    assert m == int(keep.sum())
