"""GPU parity tests: the HIP path (through the ctypes C-ABI binding) against the
CPU oracle on identical seeded inputs.

Bars: compaction indices bit-exact; loss within 1e-3 relative; grad_hidden /
grad_weight within 2e-2 relative max-norm error for bf16/f16 inputs; the
float32 cases hold the reference's own float32 tolerances (2e-5 / 3e-5,
tests/unit/kernels/test_tiled_linear_cross_entropy.py:260-300).
"""

import numpy as np
import pytest
import torch

import linear_ce_oracle as oracle
from turbo_dllm_amd import chunked_linear_ce_native as native
from turbo_dllm_amd import workloads
from turbo_dllm_amd.tiled_linear_cross_entropy import tiled_linear_cross_entropy

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-3
GRAD_REL_MAX = 2e-2


def say(*parts):
    print("[case]", *parts, flush=True)


def run_api(dev, hidden, weight, labels, *, bias=None, grad_out=None, frozen=False, **kw):
    """Loss and gradients of the device path for CPU-resident inputs."""
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(not frozen)
    b = None if bias is None else bias.to(dev).requires_grad_(True)
    loss = tiled_linear_cross_entropy(h, w, labels.to(dev), bias=b, **kw)
    go = None if grad_out is None else grad_out.to(dev)
    loss.backward(go)
    torch.cuda.synchronize()
    return (loss.detach().cpu(), h.grad.cpu(), None if frozen else w.grad.cpu(),
            None if b is None else b.grad.cpu())


def check_against_oracle(dev, hidden, weight, labels, *, bias=None, reduction="mean",
                         exclude_index=None, logit_softcap=None, weight_layout="vocab_first",
                         odtype=torch.float64, loss_rtol=LOSS_RTOL, grad_rel=GRAD_REL_MAX,
                         grad_out=None, frozen=False):
    dim_first = weight_layout == "dim_first"
    loss, dh, dw, db = run_api(dev, hidden, weight, labels, bias=bias, grad_out=grad_out,
                               frozen=frozen, reduction=reduction, exclude_index=exclude_index,
                               logit_softcap=logit_softcap, dtype=hidden.dtype,
                               weight_layout=weight_layout)
    ref = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, reduction=reduction,
                                 exclude_index=exclude_index, logit_softcap=logit_softcap,
                                 weight_dim_first=dim_first, dtype=odtype)
    assert loss.dtype == torch.float32 and loss.shape == ref.shape
    torch.testing.assert_close(loss.double(), ref.double(), rtol=loss_rtol, atol=loss_rtol * 1e-2)
    rdh, rdw, rdb = oracle.dense_linear_ce_grads(
        hidden, weight, labels, grad_out, bias=bias, reduction=reduction,
        exclude_index=exclude_index, logit_softcap=logit_softcap, weight_dim_first=dim_first,
        dtype=odtype)
    assert dh.dtype == hidden.dtype and dh.shape == hidden.shape
    errs = {"dh": oracle.relative_max_error(dh, rdh)}
    if not frozen:
        assert dw.dtype == weight.dtype and dw.shape == weight.shape
        errs["dw"] = oracle.relative_max_error(dw, rdw)
    if bias is not None:
        errs["db"] = oracle.relative_max_error(db, rdb)
    say("errors", {k: f"{v:.2e}" for k, v in errs.items()})
    for name, err in errs.items():
        assert err <= grad_rel, (name, err)
    # rows without loss get exactly zero gradient
    ignored = (labels.reshape(-1) == -100)
    if ignored.any():
        assert torch.count_nonzero(dh.reshape(-1, dh.shape[-1])[ignored]) == 0
    return loss, dh, dw, db


# ------------------------------------------------------------------ compaction --
@pytest.mark.parametrize("n,density", [(0, 0.5), (1, 1.0), (1, 0.0), (63, 0.5), (64, 0.5),
                                       (65, 0.5), (1023, 0.3), (1024, 0.3), (1025, 0.3),
                                       (32768, 0.5), (35011, 0.05), (100003, 0.0),
                                       (100003, 1.0), (262144, 0.5), (262145, 0.5),
                                       (1 << 20, 0.7), ((1 << 24) + 5, 0.31)])
def test_compaction_indices_are_bit_exact(gpu_device, n, density):
    say("compaction", n, density)
    rng = np.random.default_rng(n * 7 + int(density * 100))
    labels = rng.integers(0, 151936, size=n).astype(np.int64)
    labels[rng.random(n) >= density] = -100
    expect = oracle.compact_rows(labels, -100)
    idx, m = native.compact_rows(torch.from_numpy(labels).to(gpu_device), -100)
    assert m == expect.size and idx.dtype == torch.int64
    assert np.array_equal(idx.cpu().numpy(), expect)
    # a different ignore value, and labels that merely look negative
    labels2 = labels.copy()
    labels2[labels2 == -100] = -1
    idx2, m2 = native.compact_rows(torch.from_numpy(labels2).to(gpu_device), -100)
    assert m2 == n and np.array_equal(idx2.cpu().numpy(), np.arange(n))


@pytest.mark.parametrize("n,density", [(0, 0.5), (1, 1.0), (1, 0.0), (65, 0.5), (1025, 0.3),
                                       (32768, 0.25), (262145, 0.9), (1 << 20, 0.05),
                                       ((1 << 24) + 77, 0.5)])
@pytest.mark.parametrize("kind", ["bool", "uint8", "float"])
def test_mask_compaction_equals_torch_nonzero(gpu_device, n, density, kind):
    """The boolean-mask form of the scan (the DFlash call sites compact
    `supervised_mask`, dflash/model.py:870-871): bit-exact against torch.nonzero
    on the host, up to sizes that take the block-offset scan."""
    if kind != "bool" and n > (1 << 20):
        pytest.skip("the large size is covered once")
    say("mask compaction", n, density, kind)
    gen = torch.Generator().manual_seed(n * 3 + int(density * 100))
    keep = torch.rand(n, generator=gen) < density
    mask = {"bool": keep, "uint8": keep.to(torch.uint8) * 7, "float": keep.float() * -2.5}[kind]
    expect = torch.nonzero(keep, as_tuple=False).flatten()
    idx, m = native.compact_mask(mask.to(gpu_device))
    assert m == expect.numel() and idx.dtype == torch.int64
    assert torch.equal(idx.cpu(), expect)
    # a 2-D mask is scanned in its flattened order
    if n and n % 4 == 0:
        idx2, m2 = native.compact_mask(mask.reshape(4, -1).to(gpu_device))
        assert m2 == m and torch.equal(idx2.cpu(), expect)


def test_fused_gather_clamps_the_device_row_count(gpu_device):
    """A row count beyond the capacity (a stale or corrupt counter) must not walk
    past the index buffer: the gather treats it as the capacity."""
    dev = gpu_device
    torch.manual_seed(4)
    n, h = 200, 64
    hidden = torch.randn(n, h).bfloat16()
    labels = torch.randint(0, 50, (n,))
    labels[torch.rand(n) < 0.5] = -100
    idx, count = native.compact_rows_device(labels.to(dev), -100)
    m = int(count.item())
    keep = torch.nonzero(labels != -100).flatten()
    big = torch.tensor([10 * n], dtype=torch.long, device=dev)
    rows, targets, _ = native.gather_loss_rows(hidden.to(dev), labels.to(dev), None, idx, big,
                                               -100, capacity=m)
    assert rows.shape[0] == (m + 63) // 64 * 64
    assert torch.equal(rows[:m].cpu(), hidden[keep]) and torch.equal(targets[:m].cpu(), labels[keep])
    assert torch.count_nonzero(rows[m:].float()) == 0 and bool((targets[m:] == -100).all())
    negative = torch.tensor([-3], dtype=torch.long, device=dev)
    rows, targets, _ = native.gather_loss_rows(hidden.to(dev), labels.to(dev), None, idx, negative,
                                               -100, capacity=m)
    torch.cuda.synchronize()       # nothing gathered, nothing faulted


@pytest.mark.parametrize("row_shape,dtype", [((4096,), torch.bfloat16), ((96,), torch.bfloat16),
                                             ((33,), torch.float32), ((), torch.int64),
                                             ((7,), torch.bfloat16), ((3, 5), torch.float16)])
def test_gather_and_scatter_rows(gpu_device, row_shape, dtype):
    say("gather/scatter", row_shape, dtype)
    torch.manual_seed(1)
    n = 777
    if dtype == torch.int64:
        src = torch.randint(-5, 1000, (n, *row_shape))
    else:
        src = torch.randn(n, *row_shape).to(dtype)
    keep = torch.rand(n) < 0.4
    idx = torch.nonzero(keep).flatten()
    got = native.gather_rows(src.to(gpu_device), idx.to(gpu_device)).cpu()
    assert torch.equal(got, src.index_select(0, idx))
    back = native.scatter_rows(got.to(gpu_device), idx.to(gpu_device), n).cpu()
    expect = torch.zeros_like(src)
    expect[idx] = src[idx]
    assert torch.equal(back, expect)


def test_compact_valid_loss_rows_on_device(gpu_device):
    from turbo_dllm_amd.compaction import compact_valid_loss_rows

    torch.manual_seed(2)
    hidden = torch.randn(4, 50, 64).bfloat16().to(gpu_device).requires_grad_(True)
    labels = torch.randint(0, 100, (4, 50))
    labels[torch.rand(4, 50) < 0.6] = -100
    weights = torch.rand(4, 50)
    rows, targets, w = compact_valid_loss_rows(hidden, labels.to(gpu_device),
                                               weights.to(gpu_device), ignore_index=-100)
    keep = labels.reshape(-1) != -100
    assert torch.equal(rows.detach().cpu(), hidden.detach().cpu().reshape(-1, 64)[keep])
    assert torch.equal(targets.cpu(), labels.reshape(-1)[keep])
    assert torch.equal(w.cpu(), weights.reshape(-1)[keep])
    rows.float().sum().backward()
    grad = hidden.grad.cpu().reshape(-1, 64)
    assert torch.equal(grad[keep], torch.ones_like(grad[keep]))
    assert torch.count_nonzero(grad[~keep]) == 0


# --------------------------------------------- the reference's device test cases --
def test_float32_case_of_reference_suite(gpu_device):
    # test_tiled_linear_cross_entropy.py:260-300 (seed 51), generic float32 engine
    say("fp32 V=4097 H=33")
    torch.manual_seed(51)
    hidden = torch.randn(3, 7, 33)
    weight = torch.randn(4097, 33)
    bias = torch.randn(4097)
    labels = torch.randint(0, 4096, (3, 7))
    labels[0, 3] = -100
    labels[2, 5] = -100
    loss, dh, dw, db = run_api(gpu_device, hidden, weight, labels, bias=bias, reduction="mean",
                               exclude_index=4096, vocab_block_size=257)
    ref = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, exclude_index=4096)
    torch.testing.assert_close(loss, ref.float(), atol=2e-5, rtol=2e-5)
    rdh, rdw, rdb = oracle.dense_linear_ce_grads(hidden, weight, labels, bias=bias,
                                                 exclude_index=4096)
    torch.testing.assert_close(dh, rdh.float(), atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(dw, rdw.float(), atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(db, rdb.float(), atol=3e-5, rtol=3e-5)
    assert torch.count_nonzero(dw[4096]) == 0


def test_bfloat16_case_of_reference_suite(gpu_device):
    # test_tiled_linear_cross_entropy.py:303-354 (seed 52): MFMA engine, H=96 (K tail),
    # V=1025 (vocabulary tail), bias, excluded last column
    say("bf16 N=31 H=96 V=1025")
    torch.manual_seed(52)
    hidden = (torch.randn(31, 96) * 0.1).bfloat16()
    weight = (torch.randn(1025, 96) * 0.1).bfloat16()
    bias = (torch.randn(1025) * 0.1).bfloat16()
    labels = torch.randint(0, 1024, (31,))
    labels[::5] = -100
    loss, dh, dw, db = run_api(gpu_device, hidden, weight, labels, bias=bias, reduction="mean",
                               exclude_index=1024, dtype=torch.bfloat16,
                               weight_layout="vocab_first")
    ref = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, exclude_index=1024)
    torch.testing.assert_close(loss, ref.float(), atol=2e-5, rtol=2e-5)
    rdh, rdw, rdb = oracle.dense_linear_ce_grads(hidden, weight, labels, bias=bias,
                                                 exclude_index=1024)
    torch.testing.assert_close(dh.float(), rdh.float(), atol=2e-3, rtol=2e-2)
    torch.testing.assert_close(dw.float(), rdw.float(), atol=2e-3, rtol=2e-2)
    torch.testing.assert_close(db.float(), rdb.float(), atol=2e-3, rtol=2e-2)


def test_gemma_shape_hidden_gradient_of_reference_suite(gpu_device):
    # test_tiled_linear_cross_entropy.py:357-405 (seed 53): H=2816, V=262144, soft cap 30,
    # excluded column 4, frozen head, per-token weights through reduction "none"
    say("bf16 rows=4 H=2816 V=262144 softcap")
    torch.manual_seed(53)
    rows, hidden_size, vocab = 4, 2816, 262144
    hidden = torch.randn(rows, hidden_size).bfloat16()
    weight = (torch.randn(vocab, hidden_size) * 0.02).bfloat16()
    labels = torch.randint(0, vocab, (rows,))
    token_weights = torch.tensor([0.25, 0.75, 1.25, 2.0])
    h = hidden.to(gpu_device).requires_grad_(True)
    token_losses = tiled_linear_cross_entropy(
        h, weight.to(gpu_device), labels.to(gpu_device), reduction="none", exclude_index=4,
        logit_softcap=30.0, dtype=torch.bfloat16, weight_layout="vocab_first")
    loss = (token_losses.float() * token_weights.to(gpu_device)).sum() / rows
    loss.backward()
    ref_losses = oracle.dense_linear_ce(hidden, weight, labels, reduction="none",
                                        exclude_index=4, logit_softcap=30.0, dtype=torch.float32)
    ref = (ref_losses * token_weights).sum() / rows
    torch.testing.assert_close(loss.cpu(), ref, atol=2e-4, rtol=2e-4)
    rdh, _, _ = oracle.dense_linear_ce_grads(hidden, weight, labels, token_weights / rows,
                                             reduction="none", exclude_index=4,
                                             logit_softcap=30.0, dtype=torch.float32)
    assert torch.isfinite(h.grad).all()
    torch.testing.assert_close(h.grad.float().cpu(), rdh, atol=8e-3, rtol=4e-2)


def test_frozen_weight_case_of_reference_suite(gpu_device):
    # tests/unit/kernels/test_dflash_kl.py:163-200 shape (seed 47): N=13, H=64, V=521
    say("frozen bf16 N=13 H=64 V=521")
    torch.manual_seed(47)
    hidden = torch.randn(13, 64).bfloat16()
    weight = (torch.randn(521, 64) * 0.2).bfloat16()
    labels = torch.randint(0, 521, (13,))
    loss, dh, dw, _ = check_against_oracle(gpu_device, hidden, weight, labels, frozen=True)
    assert dw is None


# ------------------------------------------------------------- API semantics ----
@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_reductions_and_dtypes(gpu_device, reduction, dtype):
    say("reductions", reduction, dtype)
    torch.manual_seed(10)
    hidden = torch.randn(5, 60, 128).to(dtype)
    weight = (torch.randn(777, 128) * 0.1).to(dtype)
    bias = (torch.randn(777) * 0.1).to(dtype)
    labels = torch.randint(0, 777, (5, 60))
    labels[torch.rand(5, 60) < 0.3] = -100
    grad_out = torch.randn(5, 60) if reduction == "none" else torch.tensor(1.7)
    tol = dict(loss_rtol=1e-4, grad_rel=1e-4) if dtype == torch.float32 else {}
    check_against_oracle(gpu_device, hidden, weight, labels, bias=bias, reduction=reduction,
                         grad_out=grad_out, **tol)


def test_dim_first_and_non_contiguous(gpu_device):
    say("dim_first / non-contiguous")
    torch.manual_seed(11)
    base_hidden = torch.randn(2, 64, 72).bfloat16()            # H=72: K tail inside one slab
    base_labels = torch.randint(0, 300, (2, 64))
    weight = (torch.randn(72, 300) * 0.2).bfloat16()
    hidden, labels = base_hidden[:, ::2, :], base_labels[:, ::2]
    # strided views on the device, as in test_tiled_linear_cross_entropy.py:153-169
    h = base_hidden.to(gpu_device)[:, ::2, :].requires_grad_(True)
    y = base_labels.to(gpu_device)[:, ::2]
    w = weight.to(gpu_device).requires_grad_(True)
    assert not h.is_contiguous() and not y.is_contiguous()
    loss = tiled_linear_cross_entropy(h, w, y, reduction="sum", dtype=torch.bfloat16,
                                      weight_layout="dim_first")
    loss.backward()
    ref = oracle.dense_linear_ce(hidden, weight, labels, reduction="sum", weight_dim_first=True)
    rdh, rdw, _ = oracle.dense_linear_ce_grads(hidden, weight, labels, reduction="sum",
                                               weight_dim_first=True)
    torch.testing.assert_close(loss.cpu().double(), ref, rtol=LOSS_RTOL, atol=1e-5)
    assert h.grad.shape == (2, 32, 72) and w.grad.shape == (72, 300)
    assert oracle.relative_max_error(h.grad, rdh) <= GRAD_REL_MAX
    assert oracle.relative_max_error(w.grad, rdw) <= GRAD_REL_MAX
    # layout inference from shapes gives the same answer
    auto = tiled_linear_cross_entropy(h.detach(), w.detach(), y, reduction="sum",
                                      dtype=torch.bfloat16)
    assert torch.equal(auto, loss.detach())


@pytest.mark.parametrize("m,h,v,opts", [
    (300, 128, 1536, {}),
    (1000, 256, 4160, dict(bias=True, logit_softcap=5.0, exclude_index=7)),   # v % 256 != 0
    (130, 64, 640, dict(reduction="none", frozen=True)),
    (700, 192, 2048, dict(reduction="sum", panel_tiles=3, ignored=0.0)),     # several panels
])
def test_dim_first_head_is_read_in_place(gpu_device, m, h, v, opts):
    """A [H, V] head with 16-bit inputs and H, V multiples of 64 goes to the
    library as it is stored (tlce_*_dim_first, the reference's `weight_dim_first`
    flag, fused_linear_ce.cpp:104,121): same results as the oracle's dim-first
    branch, grad_weight comes back [H, V], and no [V, H] copy of the head is
    allocated on the way."""
    opts = dict(opts)
    say("dim-first in place", m, h, v, opts)
    torch.manual_seed(m + v)
    hidden = torch.randn(m, h).bfloat16()
    weight = (torch.randn(h, v) * 0.2).bfloat16()               # [H, V]
    bias = torch.randn(v).bfloat16() if opts.pop("bias", False) else None
    labels = torch.randint(0, v, (m,))
    exclude = opts.get("exclude_index")
    if exclude is not None:
        labels[labels == exclude] = exclude + 1
    labels[torch.rand(m) < opts.pop("ignored", 0.25)] = -100
    frozen = opts.pop("frozen", False)
    panel_tiles = opts.pop("panel_tiles", 0)
    reduction = opts.pop("reduction", "mean")
    assert native.dim_first_in_place(weight.to(gpu_device), True)
    assert not native.dim_first_in_place(weight.to(gpu_device), False)
    mp = -(-m // 256) * 256
    with native.panel_budget(mp * 256 * 2 * panel_tiles):
        grad_out = torch.randn(m) if reduction == "none" else None
        loss, dh, dw, db = check_against_oracle(
            gpu_device, hidden, weight, labels, bias=bias, reduction=reduction, frozen=frozen,
            weight_layout="dim_first", grad_out=grad_out, **opts)
    if not frozen:
        assert dw.shape == (h, v)
    # the same head laid out [V, H]: same tiles in the same order; only the label's logit is
    # summed in another order (a strided column instead of a row)
    vf = run_api(gpu_device, hidden, weight.t().contiguous(), labels, bias=bias, frozen=True,
                 grad_out=grad_out, reduction=reduction, dtype=torch.bfloat16,
                 weight_layout="vocab_first", **opts)
    torch.testing.assert_close(loss, vf[0], rtol=1e-5, atol=1e-5)
    # no transposed copy: the forward's peak allocation stays far below one more head
    dev = gpu_device
    x, w, y = hidden.to(dev), weight.to(dev), labels.to(dev)
    big_v = 64 * 1024
    w_big = (torch.randn(h, big_v, device=dev) * 0.2).bfloat16()
    y_big = torch.randint(0, big_v, (m,), device=dev)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    before = torch.cuda.memory_allocated(dev)
    with torch.no_grad():
        out = tiled_linear_cross_entropy(x, w_big, y_big, dtype=torch.bfloat16,
                                         weight_layout="dim_first")
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated(dev) - before
    say("peak extra bytes", extra, "head bytes", w_big.numel() * 2)
    assert bool(torch.isfinite(out)) and extra < w_big.numel() * 2 // 2


def test_dim_first_fallback_shapes_still_use_a_copy(gpu_device):
    """Shapes the in-place path does not take (float32, V not a multiple of 64) are
    re-laid once and give the oracle's results."""
    say("dim-first fallback")
    torch.manual_seed(21)
    for dtype, h, v in ((torch.float32, 64, 640), (torch.bfloat16, 128, 1000)):
        weight = (torch.randn(h, v) * 0.2).to(dtype)
        assert not native.dim_first_in_place(weight.to(gpu_device), True)
        hidden = torch.randn(90, h).to(dtype)
        labels = torch.randint(0, v, (90,))
        tol = dict(loss_rtol=1e-4, grad_rel=1e-4) if dtype == torch.float32 else {}
        check_against_oracle(gpu_device, hidden, weight, labels, weight_layout="dim_first", **tol)


def test_softcap_with_bias_and_exclusion(gpu_device):
    say("softcap + bias + exclude")
    torch.manual_seed(12)
    hidden = (torch.randn(300, 256) * 2).bfloat16()
    weight = (torch.randn(1000, 256) * 0.3).bfloat16()
    bias = torch.randn(1000).bfloat16()
    labels = torch.randint(1, 1000, (300,))
    labels[::7] = -100
    check_against_oracle(gpu_device, hidden, weight, labels, bias=bias, exclude_index=0,
                         logit_softcap=7.5, reduction="none", grad_out=torch.rand(300))


def test_empty_and_fully_ignored_inputs(gpu_device):
    say("empty / all ignored")
    torch.manual_seed(13)
    hidden = torch.randn(10, 64).bfloat16().to(gpu_device).requires_grad_(True)
    weight = torch.randn(50, 64).bfloat16().to(gpu_device).requires_grad_(True)
    labels = torch.full((10,), -100, device=gpu_device)
    none = tiled_linear_cross_entropy(hidden, weight, labels, reduction="none")
    assert none.shape == (10,) and torch.count_nonzero(none) == 0
    total = tiled_linear_cross_entropy(hidden, weight, labels, reduction="sum")
    total.backward()
    assert float(total.detach()) == 0.0
    assert torch.count_nonzero(hidden.grad) == 0 and torch.count_nonzero(weight.grad) == 0
    assert torch.isnan(tiled_linear_cross_entropy(hidden, weight, labels, reduction="mean"))
    zero = tiled_linear_cross_entropy(hidden[:0], weight, labels[:0], reduction="sum")
    assert float(zero) == 0.0


def test_mixed_devices_are_refused(gpu_device):
    hidden = torch.randn(4, 8)
    weight = torch.randn(9, 8)
    labels = torch.tensor([0, 1, 2, 3])
    with pytest.raises(RuntimeError, match="refusing to fall back"):
        tiled_linear_cross_entropy(hidden.to(gpu_device), weight, labels)
    with pytest.raises(ValueError, match="must match hidden prefix"):
        tiled_linear_cross_entropy(hidden.to(gpu_device), weight.to(gpu_device),
                                   labels[:3].to(gpu_device))


def test_c_abi_without_compaction_handles_ignored_rows(gpu_device):
    # the library itself (no row_idx) must zero ignored rows like the reference op
    say("C-ABI direct, ignored rows in place")
    torch.manual_seed(14)
    hidden = torch.randn(200, 128).bfloat16()
    weight = (torch.randn(500, 128) * 0.2).bfloat16()
    labels = torch.randint(0, 500, (200,))
    labels[::3] = -100
    dev = gpu_device
    kw = dict(row_block_size=0, ignore_index=-100, exclude_index=-1, logit_softcap=0.0,
              compute_dtype=torch.bfloat16, weight_dim_first=False)
    losses, lse, count = native.forward(hidden.to(dev), weight.to(dev), None, labels.to(dev), **kw)
    assert float(count) == float((labels != -100).sum())
    ref, ref_lse = oracle.dense_linear_ce(hidden, weight, labels, reduction="none",
                                          return_lse=True)
    torch.testing.assert_close(losses.cpu().double(), ref, rtol=LOSS_RTOL, atol=1e-5)
    torch.testing.assert_close(lse.cpu().double(), ref_lse, rtol=LOSS_RTOL, atol=1e-5)
    go = torch.ones(1, device=dev)
    dh, dw, db = native.backward(hidden.to(dev), weight.to(dev), None, labels.to(dev), lse, count,
                                 go, reduction="mean", **kw)
    rdh, rdw, _ = oracle.dense_linear_ce_grads(hidden, weight, labels, reduction="mean")
    assert oracle.relative_max_error(dh.cpu(), rdh) <= GRAD_REL_MAX
    assert oracle.relative_max_error(dw.cpu(), rdw) <= GRAD_REL_MAX
    assert torch.count_nonzero(dh.cpu()[::3]) == 0 and db.numel() == 0
    dh2, dw2, _ = native.backward_frozen_weight(hidden.to(dev), weight.to(dev), None,
                                                labels.to(dev), lse, count, go, reduction="mean",
                                                **kw)
    assert torch.equal(dh2, dh) and dw2.numel() == 0


def test_panel_count_does_not_change_results(gpu_device):
    say("panel budget sweep")
    torch.manual_seed(15)
    hidden = torch.randn(600, 256).bfloat16()
    weight = (torch.randn(3000, 256) * 0.1).bfloat16()
    labels = torch.randint(0, 3000, (600,))
    base = run_api(gpu_device, hidden, weight, labels, reduction="mean", dtype=torch.bfloat16)
    with native.panel_budget(768 * 256 * 2 * 2 * 3):   # three 256-column tiles per panel
        multi = run_api(gpu_device, hidden, weight, labels, reduction="mean",
                        dtype=torch.bfloat16)
    assert torch.equal(base[0], multi[0])
    assert torch.equal(base[2], multi[2])                      # grad_weight: same tiles, same order
    assert oracle.relative_max_error(multi[1], base[1].double()) < 1e-2   # grad_hidden: split differs


@pytest.mark.parametrize("m,h,v,panel_tiles", [
    (5, 64, 64, 0), (64, 128, 1024, 0), (100, 128, 1088, 2), (300, 256, 2048, 3),
    (513, 192, 4160, 4), (1000, 320, 1536, 0),
])
def test_direct_engine_in_place_operands(gpu_device, m, h, v, panel_tiles):
    # h % 64 == 0 and v % 64 == 0: the gradient contractions read weight, hidden and the
    # logit-gradient panel K-major (no transposed copies); m % 64 != 0 pads hidden rows,
    # v % 256 != 0 ends a panel inside a tile, panel_tiles forces several panels
    say("in-place operands", m, h, v, panel_tiles)
    torch.manual_seed(m + v)
    hidden = torch.randn(m + 7, h).bfloat16()
    weight = (torch.randn(v, h) * 0.2).bfloat16()
    labels = torch.randint(0, v, (m + 7,))
    labels[torch.randperm(m + 7)[:7]] = -100
    mp = -(-m // 256) * 256
    with native.panel_budget(mp * 256 * 2 * panel_tiles):   # 0: the library default
        check_against_oracle(gpu_device, hidden, weight, labels, reduction="mean")
        check_against_oracle(gpu_device, hidden, weight, labels, reduction="sum", frozen=True,
                             logit_softcap=4.0)


# ------------------------------------------- benchmark configurations, scaled ----
@pytest.mark.parametrize("name", list(workloads.CONFIGS))
def test_scaled_benchmark_configurations(gpu_device, name):
    wl = workloads.CONFIGS[name](seed=3, scale=16)
    say("config", name, "N", wl.n_rows, "M", wl.n_loss_rows, "H", wl.hidden.shape[1], "V",
        wl.weight.shape[0])
    check_against_oracle(gpu_device, wl.hidden, wl.weight, wl.labels,
                         logit_softcap=wl.logit_softcap, odtype=torch.float32)


def test_label_on_the_excluded_column(gpu_device):
    """A row labelled with the excluded column: the native path gives loss = lse
    (target logit 0, fused_linear_ce_cuda.cu:199-219) and no gradient on that
    column (:270-283); every other row is unaffected."""
    say("label == exclude, bias, bf16")
    gen = torch.Generator().manual_seed(77)
    n, h, v, exclude = 150, 128, 1536, 1023
    hidden = torch.randn(n, h, generator=gen).bfloat16()
    weight = (torch.randn(v, h, generator=gen) * 0.2).bfloat16()
    bias = torch.randn(v, generator=gen).bfloat16()
    labels = torch.randint(0, v, (n,), generator=gen)
    labels[labels == exclude] = 0
    labels[3] = exclude
    labels[5] = -100
    loss, dh, dw, db = run_api(gpu_device, hidden, weight, labels, bias=bias,
                               grad_out=torch.ones(n), reduction="none", exclude_index=exclude,
                               dtype=torch.bfloat16, weight_layout="vocab_first")
    ref, lse = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, reduction="none",
                                      exclude_index=exclude, return_lse=True)
    others = torch.ones(n, dtype=torch.bool)
    others[3] = False
    torch.testing.assert_close(loss[others].double(), ref[others].double(), rtol=LOSS_RTOL,
                               atol=1e-5)
    torch.testing.assert_close(loss[3].double(), lse[3].double(), rtol=LOSS_RTOL, atol=1e-5)
    rdh, rdw, rdb = oracle.dense_linear_ce_grads(hidden, weight, labels, torch.ones(n), bias=bias,
                                                 reduction="none", exclude_index=exclude)
    assert oracle.relative_max_error(dh, rdh) <= GRAD_REL_MAX
    assert oracle.relative_max_error(dw, rdw) <= GRAD_REL_MAX
    assert oracle.relative_max_error(db, rdb) <= GRAD_REL_MAX
    assert torch.count_nonzero(dw[exclude]) == 0 and float(db[exclude]) == 0.0


def test_contiguous_views_at_odd_offsets(gpu_device):
    """hidden[1:] and weight[v0:] are contiguous but, with rows that are not a
    multiple of 16 bytes long, no longer 16-byte aligned; the reference accepts
    any contiguous tensor (tiled_linear_cross_entropy.py:297-301)."""
    say("offset views, float32 H=33 and bf16 H=100")
    for dtype, h, v, tol in ((torch.float32, 33, 517, 3e-5), (torch.bfloat16, 100, 1025, GRAD_REL_MAX)):
        gen = torch.Generator().manual_seed(h)
        hidden_all = torch.randn(131, h, generator=gen).to(dtype)
        weight_all = (torch.randn(v + 3, h, generator=gen) * 0.2).to(dtype)
        labels = torch.randint(0, v, (130,), generator=gen)
        labels[::7] = -100
        dev = gpu_device
        hd = hidden_all.to(dev)[1:].requires_grad_(True)
        wd = weight_all.to(dev)[3:].requires_grad_(True)
        assert hd.is_contiguous() and wd.is_contiguous()
        assert hd.data_ptr() % 16 != 0 or wd.data_ptr() % 16 != 0
        loss = tiled_linear_cross_entropy(hd, wd, labels.to(dev), dtype=dtype,
                                          weight_layout="vocab_first")
        loss.backward()
        torch.cuda.synchronize()
        ref = oracle.dense_linear_ce(hidden_all[1:], weight_all[3:], labels)
        rdh, rdw, _ = oracle.dense_linear_ce_grads(hidden_all[1:], weight_all[3:], labels)
        torch.testing.assert_close(loss.detach().cpu().double(), ref, rtol=LOSS_RTOL, atol=1e-5)
        assert oracle.relative_max_error(hd.grad.cpu(), rdh) <= tol
        assert oracle.relative_max_error(wd.grad.cpu(), rdw) <= tol
