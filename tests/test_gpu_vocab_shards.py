"""GPU parity of the vocabulary-shard entry points (through the C ABI) against
the CPU oracle: per-shard softmax statistics, their combination into the
global loss, and the per-shard gradient contributions.

The reference's distributed test builds shards the same way
(tests/unit/parallel/test_vocab_parallel_cross_entropy*.py compare the
combined result with dense cross entropy); here the "ranks" are run one after
the other on one GPU and combined as the MAX / SUM all-reduces would.
"""

import pytest
import torch

import linear_ce_oracle as oracle
from turbo_dllm_amd import chunked_linear_ce_native as native

pytestmark = pytest.mark.gpu


def say(*parts):
    print("[case]", *parts, flush=True)


CASES = [
    # name, dtype, N, H, V, shard bounds, bias, softcap, exclude
    ("f32_generic", torch.float32, 37, 33, 301, (0, 100, 301), True, 0.0, -1),
    ("bf16_staged_h72", torch.bfloat16, 61, 72, 1025, (0, 512, 1025), False, 0.0, 600),
    ("bf16_direct", torch.bfloat16, 300, 256, 2304, (0, 1024, 2304), False, 0.0, -1),
    ("bf16_direct_softcap_bias", torch.bfloat16, 129, 128, 1536, (0, 512, 1024, 1536), True,
     5.0, 1023),
    ("f16_direct_uneven", torch.float16, 70, 64, 1000, (0, 640, 1000), False, 0.0, 0),
]


def make_case(dtype, n, h, v, bias, seed):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=gen).to(dtype)
    weight = (torch.randn(v, h, generator=gen) * (2.0 / h ** 0.5)).to(dtype)
    b = torch.randn(v, generator=gen).to(dtype) if bias else None
    labels = torch.randint(0, v, (n,), generator=gen)
    labels[torch.rand(n, generator=gen) < 0.25] = -100
    return hidden, weight, b, labels


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_shard_statistics_and_gradients(gpu_device, case):
    name, dtype, n, h, v, bounds, has_bias, softcap, exclude = case
    say(name)
    hidden, weight, bias, labels = make_case(dtype, n, h, v, has_bias, seed=len(name) + n)
    if exclude >= 0:
        labels[1] = exclude            # a label on the excluded column (and not ignored)
    labels[0] = -100
    dev = gpu_device
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    hd, ld = hidden.to(dev), labels.to(dev)
    shards = list(zip(bounds[:-1], bounds[1:]))

    got, ref = [], []
    for a, b in shards:
        wd = weight[a:b].to(dev)
        bd = None if bias is None else bias[a:b].to(dev)
        out = native.vocab_parallel_forward_local(
            hd, wd, bd, ld, vocab_start=a, ignore_index=-100, exclude_index=exclude,
            logit_softcap=softcap)
        torch.cuda.synchronize()
        got.append(tuple(t.cpu().double() for t in out))
        ref.append(oracle.vocab_shard_stats(
            hidden, weight[a:b], labels, vocab_start=a, bias=None if bias is None else bias[a:b],
            exclude_index=exclude, logit_softcap=softcap))
    for (a, b), g, r in zip(shards, got, ref):
        # the shard's own log-sum-exp, the target logits and the count
        torch.testing.assert_close(g[0] + torch.log(g[1]), r[0] + torch.log(r[1]),
                                   rtol=tol, atol=tol)
        torch.testing.assert_close(g[0], r[0], rtol=tol, atol=10 * tol)
        torch.testing.assert_close(g[2], r[2], rtol=tol, atol=10 * tol)
        assert float(g[3]) == float(r[3]) == float((labels != -100).sum())
    # combined as the all-reduces would: equals the dense loss of the whole head
    losses, lse = oracle.combine_vocab_shards(got, labels)
    dense, dense_lse = oracle.dense_linear_ce(
        hidden, weight, labels, bias=bias, reduction="none",
        exclude_index=exclude if exclude >= 0 else None, logit_softcap=softcap or None,
        return_lse=True)
    keep = labels != exclude
    torch.testing.assert_close(losses[keep], dense[keep].double(), rtol=tol, atol=tol)
    torch.testing.assert_close(lse, dense_lse.double(), rtol=tol, atol=tol)
    if exclude >= 0:
        assert torch.isinf(losses[1]) and losses[1] > 0    # lse - (-inf), as in the reference

    # gradients with the global lse: partial grad_hidden sums to the dense one,
    # grad_weight / grad_bias of the shards tile the dense ones
    for reduction in ("none", "mean"):
        gen = torch.Generator().manual_seed(3)
        go = torch.randn(n, generator=gen) if reduction == "none" else torch.tensor([1.7])
        labels_b = labels.clone()
        if exclude >= 0:
            labels_b[1] = (exclude + 1) % v           # keep the dense oracle finite
        lse_b = oracle.dense_linear_ce(
            hidden, weight, labels_b, bias=bias, reduction="none",
            exclude_index=exclude if exclude >= 0 else None, logit_softcap=softcap or None,
            return_lse=True)[1].float()
        count = torch.tensor([float((labels_b != -100).sum())])
        rdh, rdw, rdb = oracle.dense_linear_ce_grads(
            hidden, weight, labels_b, go if reduction == "none" else go.reshape(()), bias=bias,
            reduction=reduction,
            exclude_index=exclude if exclude >= 0 else None, logit_softcap=softcap or None)
        dh_sum = torch.zeros(n, h, dtype=torch.float64)
        dw_parts, db_parts = [], []
        for a, b in shards:
            wd = weight[a:b].to(dev)
            bd = None if bias is None else bias[a:b].to(dev)
            dh, dw, db = native.vocab_parallel_backward_local(
                hd, wd, bd, labels_b.to(dev), lse_b.to(dev), count.to(dev), go.to(dev),
                reduction=reduction, vocab_start=a, ignore_index=-100, exclude_index=exclude,
                logit_softcap=softcap)
            torch.cuda.synchronize()
            assert dh.dtype == dtype and dw.dtype == dtype and dw.shape == (b - a, h)
            dh_sum += dh.cpu().double()
            dw_parts.append(dw.cpu())
            db_parts.append(db.cpu())
        gtol = 2e-5 if dtype == torch.float32 else 2e-2
        err_h = oracle.relative_max_error(dh_sum, rdh)
        err_w = oracle.relative_max_error(torch.cat(dw_parts), rdw)
        say(reduction, "dh", f"{err_h:.2e}", "dw", f"{err_w:.2e}")
        assert err_h <= gtol and err_w <= gtol
        if bias is not None:
            assert oracle.relative_max_error(torch.cat(db_parts), rdb) <= gtol
        assert torch.count_nonzero(dh_sum[labels_b == -100]) == 0


def test_single_shard_equals_the_unsharded_entry_point(gpu_device):
    """vocab_start = 0 over the whole head: same lse, loss and gradients, bit for
    bit, as forward / backward of the unsharded entry points."""
    hidden, weight, _, labels = make_case(torch.bfloat16, 200, 128, 1280, False, seed=5)
    dev = gpu_device
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    kw = dict(row_block_size=0, ignore_index=-100, exclude_index=-1, logit_softcap=0.0,
              compute_dtype=torch.bfloat16, weight_dim_first=False)
    losses, lse, count = native.forward(hd, wd, None, ld, **kw)
    mx, sm, tg, cnt = native.vocab_parallel_forward_local(
        hd, wd, None, ld, vocab_start=0, ignore_index=-100, exclude_index=-1, logit_softcap=0.0)
    assert torch.equal(cnt, count)
    torch.testing.assert_close(mx + torch.log(sm), lse, rtol=1e-6, atol=1e-6)
    valid = ld != -100
    torch.testing.assert_close((mx + torch.log(sm) - tg)[valid], losses[valid],
                               rtol=1e-6, atol=1e-5)
    go = torch.ones(1, device=dev)
    a = native.backward(hd, wd, None, ld, lse, count, go, reduction="mean", **kw)
    b = native.vocab_parallel_backward_local(
        hd, wd, None, ld, lse, count, go, reduction="mean", vocab_start=0, ignore_index=-100,
        exclude_index=-1, logit_softcap=0.0)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
