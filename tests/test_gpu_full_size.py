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


# ------------------------------------------------- remaining configurations ----
def check_configuration_full_size(dev, wl, *, loss_rows=768, check_column_sums=True):
    """One benchmark configuration at full size against the oracle by sampling:
    per-row losses and grad_hidden rows depend on their own row only, so sampled
    rows are checked completely; grad_weight rows need every loss-bearing row but
    only their own vocabulary column, with lse_r = loss_r + target_r taken from
    the device's losses (themselves checked on the sample) and the oracle's
    target logits."""
    n, m = wl.n_rows, wl.n_loss_rows
    h, v = wl.hidden.shape[1], wl.weight.shape[0]
    cap = wl.logit_softcap
    say(wl.name, "N", n, "M", m, "H", h, "V", v, "softcap", cap)
    losses, dh, dw = run(dev, wl)
    say("device done")
    keep = wl.labels != -100
    rows = torch.nonzero(keep).flatten()
    assert torch.count_nonzero(losses[~keep]) == 0
    assert torch.count_nonzero(dh[~keep]) == 0
    assert bool(torch.isfinite(losses).all()) and bool(torch.isfinite(dh.float()).all())
    assert bool(torch.isfinite(dw.float()).all())

    gen = torch.Generator().manual_seed(1)
    sample = rows[torch.randperm(m, generator=gen)[:min(loss_rows, m)]]
    ref_loss, _ = oracle_lse_in_chunks(wl, sample)
    torch.testing.assert_close(losses[sample], ref_loss, rtol=1e-3, atol=1e-4)
    say("losses on", sample.numel(), "sampled rows ok")

    pick = sample[:32]
    rdh, _, _ = oracle.dense_linear_ce_grads(
        wl.hidden[pick], wl.weight, wl.labels[pick], torch.full((pick.numel(),), 1.0 / m),
        reduction="none", logit_softcap=cap, dtype=torch.float32)
    err = oracle.relative_max_error(dh[pick], rdh)
    say("grad_hidden sampled rows rel max err", f"{err:.2e}")
    assert err <= 2e-2

    # grad_weight on sampled vocabulary rows (some of them label rows, the first and the last)
    vs = torch.cat([torch.randint(0, v, (22,), generator=gen), wl.labels[rows[:8]],
                    torch.tensor([0, v - 1])])
    h32 = wl.hidden[rows].float()
    y = wl.labels[rows]
    target = (h32 * wl.weight[y].float()).sum(dim=1)
    if cap:
        target = torch.tanh(target / cap) * cap
    lse = losses[rows] + target
    z = h32 @ wl.weight[vs].float().t()
    dcap = 1.0
    if cap:
        t = torch.tanh(z / cap)
        z, dcap = t * cap, 1.0 - t * t
    g = (torch.exp(z - lse[:, None]) - (y[:, None] == vs[None, :]).float()) * dcap / m
    rdw = g.t() @ h32
    err = oracle.relative_max_error(dw[vs], rdw)
    say("grad_weight sampled rows rel max err", f"{err:.2e}")
    assert err <= 2e-2

    lhs = float((dw.double() * wl.weight.double()).sum())
    rhs = float((dh.double() * wl.hidden.double()).sum())
    say("inner products", lhs, rhs)
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs))
    if check_column_sums:      # sum_v g[r, v] = 0 holds only without the cap's derivative
        col = dw.double().sum(dim=0).abs()
        scale = dw.double().abs().sum(dim=0)
        assert float((col / scale).max()) <= 2e-2


def test_block_diffusion_shard_full_size(gpu_device):
    check_configuration_full_size(gpu_device, workloads.block_diffusion_shard(seed=6))


def test_gemma_softcap_head_full_size(gpu_device):
    # H=3840, V=262144 (1024 vocabulary tiles, four panels), soft cap 30
    check_configuration_full_size(gpu_device, workloads.gemma_softcap_head(seed=7),
                                  loss_rows=512, check_column_sums=False)


def test_sparse_drafter_head_full_size(gpu_device):
    # ~35k rows of which ~1.8k bear loss, Zipf labels: small M, split-K grad_hidden
    from turbo_dllm_amd import _lib
    wl = workloads.sparse_drafter_head(seed=8)
    plan = _lib.query_plan(wl.n_loss_rows, 4096, 151936, _lib.DTYPE_BF16, True)
    say("plan", plan)
    assert plan["grad_hidden_k_splits"] > 1
    check_configuration_full_size(gpu_device, wl, loss_rows=4096)


def test_block_diffusion_shard_full_size_without_host_read_back(gpu_device):
    """The same configuration through the masked-token loss with the row count
    kept on the device: launches are sized for all 32768 rows, ~8.3k are real."""
    from turbo_dllm_amd.layers import VocabParallelLinear
    from turbo_dllm_amd.loss import masked_token_loss
    from turbo_dllm_amd.tiled_linear_cross_entropy import compaction_mode

    dev = gpu_device
    wl = workloads.block_diffusion_shard(seed=9)
    n, m = wl.n_rows, wl.n_loss_rows
    say("masked_token_loss, device row count: N", n, "M", m)
    head = VocabParallelLinear(4096, 151936, bias=False).to(device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        head.weight.copy_(wl.weight.to(dev))
    gen = torch.Generator().manual_seed(2)
    weights = torch.rand(n, generator=gen) + 0.5
    results = {}
    for mode in ("sync", "device"):
        hidden = wl.hidden.to(dev).requires_grad_(True)
        head.weight.grad = None
        with compaction_mode(mode):
            loss = masked_token_loss(hidden, wl.labels.to(dev), weights.to(dev), head,
                                     valid_token_count=float(m), mask_token_id=5,
                                     output_multiplier=0.5, loss_scale=2.0)
            loss.backward()
        torch.cuda.synchronize()
        results[mode] = (loss.detach().cpu(), hidden.grad.cpu(), head.weight.grad.cpu())
        say(mode, "loss", float(loss.detach()))
    # same forward plan in both modes -> identical loss; gradients differ only in the
    # order the vocabulary panels are accumulated
    assert torch.equal(results["sync"][0], results["device"][0])
    for a, b in zip(results["sync"][1:], results["device"][1:]):
        assert oracle.relative_max_error(b, a.float()) <= 5e-3
    keep = wl.labels != -100
    rows = torch.nonzero(keep).flatten()
    pick = rows[torch.randperm(m, generator=gen)[:256]]
    labels = wl.labels.clone()
    ref = oracle.masked_token_loss(wl.hidden[pick], wl.weight, labels[pick], weights[pick],
                                   float(m), exclude_index=5, output_multiplier=0.5,
                                   loss_scale=2.0, dtype=torch.float32)
    rdh, _, _ = oracle.masked_token_loss_grads(wl.hidden[pick], wl.weight, labels[pick],
                                               weights[pick], float(m), exclude_index=5,
                                               output_multiplier=0.5, loss_scale=2.0,
                                               dtype=torch.float32)
    loss, dh, dw = results["device"]
    err = oracle.relative_max_error(dh[pick], rdh)
    say("grad_hidden sampled rows rel max err", f"{err:.2e}", "sample loss share", float(ref))
    assert err <= 2e-2
    assert torch.count_nonzero(dh[~keep]) == 0 and torch.count_nonzero(dw[5]) == 0
    lhs = float((dw.double() * wl.weight.double()).sum())
    rhs = float((dh.double() * wl.hidden.double()).sum())
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs))


# --------------------------------------- the other objectives at their bench shapes ----
def _randn(gen, rows, cols, std, dev=None):
    t = (torch.randn(rows, cols, generator=gen) * std).bfloat16()
    return t if dev is None else t.to(dev)


def test_frozen_kl_full_size(gpu_device):
    from turbo_dllm_amd.dflash_kl import frozen_linear_kl

    dev = gpu_device
    m, h, v = 8192, 4096, 151936
    say("frozen-head KL M", m, "H", h, "V", v)
    gen = torch.Generator().manual_seed(11)
    dw, tw = _randn(gen, v, h, 0.02), _randn(gen, v, h, 0.02)
    dh, th = _randn(gen, m, h, 1.0), _randn(gen, m, h, 1.0)
    scale = torch.rand(m, generator=gen) + 0.5
    x = dh.to(dev).requires_grad_(True)
    got = frozen_linear_kl(x, dw.to(dev), th.to(dev), tw.to(dev))
    (got * scale.to(dev)).sum().backward()
    torch.cuda.synchronize()
    say("device done")
    got, grad = got.detach().cpu(), x.grad.cpu()
    assert bool(torch.isfinite(got).all()) and bool((got > -1e-3).all())
    pick = torch.randperm(m, generator=gen)[:48]
    ref = oracle.dense_frozen_kl(dh[pick], dw, th[pick], tw, dtype=torch.float32)
    ref_grad = oracle.dense_frozen_kl_grad(dh[pick], dw, th[pick], tw, scale[pick],
                                           dtype=torch.float32)
    say("loss max abs err", float((got[pick] - ref).abs().max()), "ref max", float(ref.max()))
    torch.testing.assert_close(got[pick], ref, rtol=2e-2, atol=2e-2)   # the reference's KL bar
    err = oracle.relative_max_error(grad[pick], ref_grad)
    say("grad rel max err", f"{err:.2e}")
    assert err <= 4e-2


def test_ce_topk_full_size(gpu_device):
    # V = 151936 is more than nine 16384-logit chunks per row: the multi-chunk scan
    from turbo_dllm_amd.dflash_linear_topk import frozen_linear_ce_topk

    dev = gpu_device
    m, h, v, k = 8192, 4096, 151936, 16
    say("CE + top-k M", m, "H", h, "V", v, "k", k)
    gen = torch.Generator().manual_seed(12)
    weight, hidden = _randn(gen, v, h, 0.02), _randn(gen, m, h, 1.0)
    labels = torch.randint(0, v, (m,), generator=gen)
    gl, gp, gv = (torch.randn(m, generator=gen), torch.randn(m, generator=gen),
                  torch.randn(m, k, generator=gen))
    x = hidden.to(dev).requires_grad_(True)
    loss, prob, vals, ids = frozen_linear_ce_topk(x, weight.to(dev), labels.to(dev), top_k=k)
    ((gl.to(dev) * loss).sum() + (gp.to(dev) * prob).sum() + (gv.to(dev) * vals).sum()).backward()
    torch.cuda.synchronize()
    say("device done")
    loss, prob, vals, ids, grad = (t.detach().cpu() for t in (loss, prob, vals, ids, x.grad))
    assert bool((vals[:, :-1] >= vals[:, 1:]).all())
    assert bool(((ids >= 0) & (ids < v)).all())
    pick = torch.randperm(m, generator=gen)[:48]
    r_loss, r_prob, r_vals, r_ids, _ = oracle.dense_ce_topk(hidden[pick], weight, labels[pick], k,
                                                            dtype=torch.float32)
    torch.testing.assert_close(loss[pick], r_loss, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(prob[pick], r_prob, rtol=2e-3, atol=1e-4)
    torch.testing.assert_close(vals[pick], r_vals, rtol=1e-3, atol=1e-3)
    agree = float((ids[pick] == r_ids).double().mean())
    say("ids agreeing with the oracle", agree)
    assert agree > 0.97
    r_grad = oracle.dense_ce_topk_grad(hidden[pick], weight, labels[pick], ids[pick], gl[pick],
                                       gp[pick], gv[pick], dtype=torch.float32)
    err = oracle.relative_max_error(grad[pick], r_grad)
    say("grad rel max err", f"{err:.2e}")
    assert err <= 2e-2


def test_soft_embedding_full_size(gpu_device):
    from turbo_dllm_amd.streaming_soft_embedding import streaming_soft_embedding

    dev = gpu_device
    m, h, v = 8192, 3840, 262144
    say("soft embedding M", m, "H", h, "V", v, "softcap 30")
    gen = torch.Generator().manual_seed(13)
    weight, hidden = _randn(gen, v, h, 0.02), _randn(gen, m, h, 1.0)
    out = streaming_soft_embedding(hidden.to(dev), weight.to(dev), row_chunk_size=1024,
                                   vocab_chunk_size=8192, logit_softcap=30.0,
                                   embedding_scale=62.0)
    torch.cuda.synchronize()
    say("device done")
    out = out.cpu()
    assert out.shape == (m, h) and bool(torch.isfinite(out.float()).all())
    pick = torch.randperm(m, generator=gen)[:48]
    ref = oracle.dense_soft_embedding(hidden[pick], weight, logit_softcap=30.0,
                                      embedding_scale=62.0, dtype=torch.float32)
    err = oracle.relative_max_error(out[pick], ref)
    say("rel max err", f"{err:.2e}")
    assert err <= 2e-2


def test_small_head_full_size_against_the_dense_oracle(gpu_device):
    """The CPU-runnable configuration (2048 rows, H=1024, V=32000, half the rows
    loss-bearing) at full size: the whole loss and both gradients against the
    dense float32 oracle."""
    wl = workloads.small_head(seed=14)
    say(wl.name, "N", wl.n_rows, "M", wl.n_loss_rows)
    hidden = wl.hidden.to(gpu_device).requires_grad_(True)
    weight = wl.weight.to(gpu_device).requires_grad_(True)
    loss = tiled_linear_cross_entropy(hidden, weight, wl.labels.to(gpu_device), reduction="mean",
                                      dtype=torch.bfloat16, weight_layout="vocab_first")
    loss.backward()
    torch.cuda.synchronize()
    ref = oracle.dense_linear_ce(wl.hidden, wl.weight, wl.labels, dtype=torch.float32)
    rdh, rdw, _ = oracle.dense_linear_ce_grads(wl.hidden, wl.weight, wl.labels,
                                               dtype=torch.float32)
    rel = abs(float(loss.detach()) - float(ref)) / abs(float(ref))
    err_h = oracle.relative_max_error(hidden.grad.cpu(), rdh)
    err_w = oracle.relative_max_error(weight.grad.cpu(), rdw)
    say(f"loss rel {rel:.2e} dH {err_h:.2e} dW {err_w:.2e}")
    assert rel <= 1e-3 and err_h <= 2e-2 and err_w <= 2e-2
