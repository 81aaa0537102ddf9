"""The allocation-free forward entry point (tlce_forward_noalloc) against
tlce_forward, through the C ABI.

Both run the same kernels; the only difference is where the per-split softmax
partials live (a static device array instead of a caller workspace), so the
results must be bit-identical: losses, lse and the valid-row count.  Two calls
in a row, the second on a smaller input, show that the shared array's leftover
contents do not leak into a later call.  The oracle bounds both (loss within
1e-3 relative).
"""

import pytest
import torch

import linear_ce_oracle as oracle
from turbo_dllm_amd import _lib
from turbo_dllm_amd import chunked_linear_ce_native as native

LOSS_RTOL = 1e-3


def _case(seed, n, h, v, dtype, ignore_every):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=gen).to(dtype)
    weight = (torch.randn(v, h, generator=gen) * 0.1).to(dtype)
    labels = torch.randint(0, v, (n,), generator=gen)
    labels[::ignore_every] = -100
    return hidden, weight, labels


def _forward_noalloc(dev, hidden, weight, labels, softcap=0.0, exclude=-1):
    lib = _lib.library()
    m, h = hidden.shape
    v = weight.shape[0]
    losses = torch.full((m,), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((m,), float("nan"), dtype=torch.float32, device=dev)
    count = torch.full((1,), float("nan"), dtype=torch.float32, device=dev)
    code = native._dtype_code(hidden)
    stream = torch.cuda.current_stream(dev).cuda_stream
    rc = lib.tlce_forward_noalloc(
        hidden.data_ptr(), weight.data_ptr(), None, labels.data_ptr(), None,
        m, m, h, v, code, -100, exclude, float(softcap),
        losses.data_ptr(), lse.data_ptr(), count.data_ptr(), stream)
    _lib.check(rc, "tlce_forward_noalloc")
    return losses, lse, count


@pytest.mark.gpu
def test_noalloc_forward_matches_workspace_forward_twice(gpu_device):
    dev = gpu_device
    kw = dict(row_block_size=0, ignore_index=-100, exclude_index=-1, logit_softcap=0.0,
              compute_dtype=torch.bfloat16, weight_dim_first=False)
    # a larger call first (several token tiles and vocabulary splits), then a
    # smaller one that reuses the front of the same static array
    for seed, n, h, v, dtype in ((71, 1100, 256, 5000, torch.bfloat16),
                                 (72, 300, 128, 777, torch.bfloat16),
                                 (73, 130, 33, 517, torch.float32)):
        print(f"[case] noalloc forward seed={seed} n={n} h={h} v={v} {dtype}", flush=True)
        hidden, weight, labels = _case(seed, n, h, v, dtype, 3)
        hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
        kw["compute_dtype"] = dtype
        want_losses, want_lse, want_count = native.forward(hd, wd, None, ld, **kw)
        got_losses, got_lse, got_count = _forward_noalloc(dev, hd, wd, ld)
        torch.cuda.synchronize()
        assert torch.equal(got_losses, want_losses)
        assert torch.equal(got_lse, want_lse)
        assert torch.equal(got_count, want_count)
        ref = oracle.dense_linear_ce(hidden, weight, labels, reduction="none")
        torch.testing.assert_close(got_losses.cpu().double(), ref, rtol=LOSS_RTOL, atol=1e-5)
        assert float(got_count) == float((labels != -100).sum())


@pytest.mark.gpu
def test_noalloc_forward_with_softcap_and_excluded_column(gpu_device):
    dev = gpu_device
    hidden, weight, labels = _case(74, 513, 192, 2049, torch.bfloat16, 5)
    labels[labels == 4] = 5
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    want = native.forward(hd, wd, None, ld, row_block_size=0, ignore_index=-100, exclude_index=4,
                          logit_softcap=30.0, compute_dtype=torch.bfloat16,
                          weight_dim_first=False)
    got = _forward_noalloc(dev, hd, wd, ld, softcap=30.0, exclude=4)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_noalloc_forward_rejects_sizes_beyond_the_static_array():
    # the size check comes first and touches no GPU: fake (aligned) pointers are never used
    lib = _lib.library()
    too_many = 524288 + 1
    rc = lib.tlce_forward_noalloc(4096, 8192, None, 12288, None, too_many, too_many, 64, 1000,
                                  _lib.DTYPE_BF16, -100, -1, 0.0, 16384, 20480, 24576, None)
    assert rc != 0
    message = _lib.last_error()
    assert "static scratch" in message and "524288" in message
    assert lib.tlce_forward_workspace_bytes(524288, 64, 1000, _lib.DTYPE_BF16) == 4 << 20
    assert lib.tlce_forward_workspace_bytes(too_many, 64, 1000, _lib.DTYPE_BF16) > 4 << 20
