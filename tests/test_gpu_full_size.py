"""Full-size GPU checks at H=4096, V=151936 through properties that do not need
a dense oracle over every row and column.

  * every per-row loss against the float32 oracle computed in row chunks;
  * grad_hidden on sampled rows and grad_weight on sampled vocabulary rows
    against the oracle formula (each depends on one row / one column only), with
    the oracle's lse over every loss-bearing row - also at the shape the
    benchmark times (32768 loss-bearing rows);
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


def run(dev, wl, grad_scale=1.0, reduction="none", gradients=None):
    """Forward + backward through the public operator.  gradients: the gradient mode
    (options.GRADIENT_MODES); by default reduction "none" is run through the backward
    that recomputes the logits and "mean" through the forward that forms the gradients
    while the logits exist, so that the tests below cover both at full size."""
    from turbo_dllm_amd import options
    if gradients is None:
        gradients = "recompute" if reduction == "none" else "forward"
    hidden = wl.hidden.to(dev).requires_grad_(True)
    weight = wl.weight.to(dev).requires_grad_(True)
    with options.gradient_mode(gradients):
        losses = tiled_linear_cross_entropy(hidden, weight, wl.labels.to(dev),
                                            reduction=reduction, logit_softcap=wl.logit_softcap,
                                            dtype=hidden.dtype, weight_layout="vocab_first")
    m = max(wl.n_loss_rows, 1)
    if reduction == "none":
        losses.backward(torch.full_like(losses, grad_scale / m))
    else:
        (losses * grad_scale).backward()
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
    check_configuration_full_size(gpu_device, workloads.qwen3_8b_head(seed=5))


def test_headline_shape_against_oracle(gpu_device):
    """The shape the benchmark times (32768 loss-bearing rows, ten vocabulary
    panels, float32 grad_hidden accumulation over ten passes): every loss, sampled
    grad_hidden rows and sampled grad_weight rows against the float32 oracle with
    the oracle's own lse, then the size-independent properties."""
    wl = workloads.block_diffusion_shard(seed=0, all_rows_loss_bearing=True)
    n = wl.n_rows
    v = wl.weight.shape[0]
    plan_columns = 16384           # width of a vocabulary panel at this shape
    gen = torch.Generator().manual_seed(2)
    # token rows at the 256-row tile edges and random ones; vocabulary rows at both ends,
    # on either side of the first and the last panel boundary, random ones and labels
    token_rows = torch.cat([torch.tensor([0, 255, 256, 16383, 16384, n - 257, n - 256, n - 1]),
                            torch.randperm(n, generator=gen)[:40]])
    last_panel = (v // plan_columns) * plan_columns
    vocab_rows = torch.cat([torch.tensor([0, 1, plan_columns - 1, plan_columns, plan_columns + 1,
                                          last_panel - 1, last_panel, v - 256, v - 1]),
                            torch.randint(0, v, (31,), generator=gen)])
    losses, dh, dw = check_configuration_full_size(gpu_device, wl, token_rows=token_rows,
                                                   vocab_rows=vocab_rows)
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
def check_configuration_full_size(dev, wl, *, check_column_sums=True, token_rows=None,
                                  vocab_rows=None, reduction="none", gradients=None):
    """One benchmark configuration at full size against the float32 oracle.

    The oracle's per-row loss and lse are computed for every loss-bearing row (in
    row chunks), so every loss is compared.  A grad_hidden row depends on its own
    row only: sampled rows are checked completely.  A grad_weight row needs every
    loss-bearing row but only its own vocabulary column: sampled vocabulary rows
    (both ends, label rows, random ones) are formed from the oracle's lse over
    all rows.  Nothing on the reference side of a comparison comes from the
    device."""
    n, m = wl.n_rows, wl.n_loss_rows
    h, v = wl.hidden.shape[1], wl.weight.shape[0]
    cap = wl.logit_softcap
    say(wl.name, "N", n, "M", m, "H", h, "V", v, "softcap", cap)
    losses, dh, dw = run(dev, wl, reduction=reduction, gradients=gradients)
    say("device done")
    keep = wl.labels != -100
    rows = torch.nonzero(keep).flatten()
    assert torch.count_nonzero(dh[~keep]) == 0
    assert bool(torch.isfinite(losses).all()) and bool(torch.isfinite(dh.float()).all())
    assert bool(torch.isfinite(dw.float()).all())

    ref_loss, ref_lse = oracle_lse_in_chunks(wl, rows)
    if reduction == "none":
        assert torch.count_nonzero(losses[~keep]) == 0
        torch.testing.assert_close(losses[rows], ref_loss, rtol=1e-3, atol=1e-4)
        say("losses on all", rows.numel(), "loss-bearing rows ok")
    else:
        ref_mean = float(ref_loss.double().mean())
        say("mean loss", float(losses), "oracle", ref_mean)
        assert abs(float(losses) - ref_mean) <= 1e-3 * abs(ref_mean)

    gen = torch.Generator().manual_seed(1)
    if token_rows is None:
        token_rows = rows[torch.randperm(m, generator=gen)[:32]]
    rdh, _, _ = oracle.dense_linear_ce_grads(
        wl.hidden[token_rows], wl.weight, wl.labels[token_rows],
        torch.full((token_rows.numel(),), 1.0 / m),
        reduction="none", logit_softcap=cap, dtype=torch.float32)
    err = oracle.relative_max_error(dh[token_rows], rdh)
    say("grad_hidden on", token_rows.numel(), "sampled rows rel max err", f"{err:.2e}")
    assert err <= 2e-2

    if vocab_rows is None:
        vocab_rows = torch.cat([torch.randint(0, v, (22,), generator=gen), torch.tensor([0, v - 1])])
    vs = torch.cat([vocab_rows, wl.labels[rows[:8]]])     # some of them label rows
    h32 = wl.hidden[rows].float()
    y = wl.labels[rows]
    z = h32 @ wl.weight[vs].float().t()
    dcap = 1.0
    if cap:
        t = torch.tanh(z / cap)
        z, dcap = t * cap, 1.0 - t * t
    g = (torch.exp(z - ref_lse[:, None]) - (y[:, None] == vs[None, :]).float()) * dcap / m
    rdw = g.t() @ h32
    err = oracle.relative_max_error(dw[vs], rdw)
    say("grad_weight on", vs.numel(), "sampled vocabulary rows rel max err", f"{err:.2e}")
    assert err <= 2e-2

    lhs = float((dw.double() * wl.weight.double()).sum())
    rhs = float((dh.double() * wl.hidden.double()).sum())
    say("inner products", lhs, rhs)
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs))
    if check_column_sums:      # sum_v g[r, v] = 0 holds only without the cap's derivative
        col = dw.double().sum(dim=0).abs()
        scale = dw.double().abs().sum(dim=0)
        assert float((col / scale).max()) <= 2e-2
    return losses, dh, dw


def test_block_diffusion_shard_full_size(gpu_device):
    check_configuration_full_size(gpu_device, workloads.block_diffusion_shard(seed=6))


# The same configurations with the loss reduced to its mean: the gradients are formed
# in the forward, in blocks of rows over the whole vocabulary (three contractions).
def test_headline_shape_gradients_formed_in_the_forward(gpu_device):
    """The shape and path the benchmark times: 32768 loss-bearing rows in four blocks
    of 8192, grad_weight accumulated in float32 over the blocks.  Token rows on block
    and tile edges, vocabulary rows at both ends, labels and random ones."""
    from turbo_dllm_amd import _lib
    wl = workloads.block_diffusion_shard(seed=0, all_rows_loss_bearing=True)
    n, v = wl.n_rows, wl.weight.shape[0]
    plan = _lib.query_fused_plan(n, 4096, v, _lib.DTYPE_BF16)
    say("plan", plan)
    block_rows = plan["block_rows"]
    assert plan["n_blocks"] == 4 and block_rows == 8192
    gen = torch.Generator().manual_seed(3)
    token_rows = torch.cat([torch.tensor([0, 255, 256, block_rows - 1, block_rows,
                                          3 * block_rows - 1, 3 * block_rows, n - 1]),
                            torch.randperm(n, generator=gen)[:40]])
    vocab_rows = torch.cat([torch.tensor([0, 1, 255, 256, v - 256, v - 1]),
                            torch.randint(0, v, (34,), generator=gen)])
    _, dh, dw = check_configuration_full_size(gpu_device, wl, token_rows=token_rows,
                                              vocab_rows=vocab_rows, reduction="mean")
    _, dh2, dw2 = run(gpu_device, wl, grad_scale=2.0, reduction="mean")
    assert torch.equal(dh2.float(), dh.float() * 2.0)
    assert torch.equal(dw2.float(), dw.float() * 2.0)


def test_headline_shape_in_one_block_with_a_panel_beyond_2_31_entries(gpu_device):
    """A panel budget that lets all 32768 rows form one block: the panel then has
    4.98e9 entries (9.96 GB), so every row offset into it must be formed in 64 bits,
    and the grad_weight contraction is the one postponed to the backward.  Compared on
    every entry with the default plan (four blocks), which the test above holds to the
    oracle: the two differ only by where sums are rounded."""
    from turbo_dllm_amd import _lib, options
    wl = workloads.block_diffusion_shard(seed=0, all_rows_loss_bearing=True)
    n, v = wl.n_rows, wl.weight.shape[0]
    budget = 10 << 30
    plan = _lib.query_fused_plan(n, 4096, v, _lib.DTYPE_BF16, budget)
    say("plan", plan)
    assert plan["n_blocks"] == 1 and plan["block_rows"] * v > 2 ** 31
    with options.panel_budget(budget):
        loss1, dh1, dw1 = run(gpu_device, wl, reduction="mean")
    loss4, dh4, dw4 = run(gpu_device, wl, reduction="mean")
    say("mean loss", float(loss1), float(loss4))
    assert abs(float(loss1) - float(loss4)) <= 1e-5 * abs(float(loss4))
    assert bool(torch.isfinite(dh1.float()).all()) and bool(torch.isfinite(dw1.float()).all())
    err_h = oracle.relative_max_error(dh1, dh4.float())
    err_w = oracle.relative_max_error(dw1, dw4.float())
    say("one block against four: grad_hidden", f"{err_h:.2e}", "grad_weight", f"{err_w:.2e}")
    assert err_h <= 1e-2 and err_w <= 1e-2
    # the last rows and the last vocabulary rows sit at the largest offsets
    assert oracle.relative_max_error(dh1[-256:], dh4[-256:].float()) <= 1e-2
    assert oracle.relative_max_error(dw1[-256:], dw4[-256:].float()) <= 1e-2


def test_block_diffusion_shard_full_size_gradients_formed_in_the_forward(gpu_device):
    check_configuration_full_size(gpu_device, workloads.block_diffusion_shard(seed=6),
                                  reduction="mean")


def test_block_diffusion_shard_full_size_per_token_losses_gradients_formed_in_the_forward(
        gpu_device):
    """Per-token losses (reduction "none") as the reference's call sites ask for them:
    one block of rows, grad_hidden rows scaled in the backward, grad_weight contracted
    there from the panel the forward left."""
    check_configuration_full_size(gpu_device, workloads.block_diffusion_shard(seed=6),
                                  reduction="none", gradients="forward")


def test_gemma_softcap_head_full_size_gradients_formed_in_the_forward(gpu_device):
    check_configuration_full_size(gpu_device, workloads.gemma_softcap_head(seed=7),
                                  check_column_sums=False, reduction="mean")


def test_sparse_drafter_head_full_size_gradients_formed_in_the_forward(gpu_device):
    check_configuration_full_size(gpu_device, workloads.sparse_drafter_head(seed=8),
                                  reduction="mean")


def test_gemma_softcap_head_full_size(gpu_device):
    # H=3840, V=262144 (1024 vocabulary tiles, four panels), soft cap 30
    check_configuration_full_size(gpu_device, workloads.gemma_softcap_head(seed=7),
                                  check_column_sums=False)


def test_sparse_drafter_head_full_size(gpu_device):
    # ~35k rows of which ~1.8k bear loss, Zipf labels: small M, split-K grad_hidden
    from turbo_dllm_amd import _lib
    wl = workloads.sparse_drafter_head(seed=8)
    plan = _lib.query_plan(wl.n_loss_rows, 4096, 151936, _lib.DTYPE_BF16, True)
    say("plan", plan)
    assert plan["grad_hidden_k_splits"] > 1
    check_configuration_full_size(gpu_device, wl)


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
    # "sync" forms the gradients in the forward (three contractions), "device" in a
    # backward that recomputes the logits: the same loss up to summation order, and
    # gradients that differ by the rounding of two different 16-bit panels
    torch.testing.assert_close(results["sync"][0], results["device"][0], rtol=1e-5, atol=0)
    for a, b in zip(results["sync"][1:], results["device"][1:]):
        assert oracle.relative_max_error(b, a.float()) <= 1e-2
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


def test_row_blocks_of_the_objectives_whose_gradient_is_formed_in_the_forward(gpu_device):
    """12000 rows at V = 151936 exceed one block of the panel budget (8192 rows): the KL
    and the cross entropy with top-k take them as two blocks, each a call of its own on a
    part of every per-row buffer.  Rows are independent, so the result equals, bit for
    bit, the two parts run on their own (which the smaller tests hold to the oracle)."""
    from turbo_dllm_amd import _lib
    from turbo_dllm_amd.dflash_kl import frozen_linear_kl
    from turbo_dllm_amd.dflash_linear_topk import frozen_linear_ce_topk
    dev = gpu_device
    m, h, v, k = 12000, 256, 151936, 4
    block = _lib.query_fused_plan(m, h, v, _lib.DTYPE_BF16, 0)["block_rows"]
    say("row blocks", m, "rows in blocks of", block)
    assert 0 < block < m
    gen = torch.Generator().manual_seed(12)
    draft_h, teacher_h = _randn(gen, m, h, 1.0, dev), _randn(gen, m, h, 1.0, dev)
    draft_w, teacher_w = _randn(gen, v, h, 0.05, dev), _randn(gen, v, h, 0.05, dev)
    labels = torch.randint(0, v, (m,), generator=gen).to(dev)
    go = (torch.rand(m, generator=gen) + 0.5).to(dev)

    def kl(rows):
        x = draft_h[rows].clone().requires_grad_(True)
        loss = frozen_linear_kl(x, draft_w, teacher_h[rows], teacher_w)
        loss.backward(go[rows])
        return loss.detach(), x.grad

    def topk(rows):
        x = draft_h[rows].clone().requires_grad_(True)
        loss, prob, vals, ids = frozen_linear_ce_topk(x, draft_w, labels[rows], top_k=k)
        (loss * go[rows]).sum().backward()
        return loss.detach(), vals.detach(), ids, x.grad

    for name, fn in (("KL", kl), ("CE top-k", topk)):
        whole = fn(slice(0, m))
        parts = [fn(slice(0, block)), fn(slice(block, m))]
        torch.cuda.synchronize()
        for i, out in enumerate(whole):
            assert bool(torch.isfinite(out.float()).all()) if out.is_floating_point() else True
            assert torch.equal(out, torch.cat([parts[0][i], parts[1][i]])), (name, i)
        say(name, "two blocks equal the parts run alone")
