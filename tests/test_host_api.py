"""CPU tests of the loss API: dispatch, layout inference, error behaviour and
the host-tensor implementation.

The cases re-create the reference's own CPU unit tests
(tests/unit/kernels/test_tiled_linear_cross_entropy.py:15-257, :408-453) with
the same seeds, shapes, tile sizes and tolerances; the expected values come
from the oracle (pinned in test_oracle_pins.py) and from F.cross_entropy.
"""

import subprocess
import sys
from pathlib import Path

import pytest
import torch
import torch.nn.functional as F

import linear_ce_oracle as oracle
from turbo_dllm_amd.tiled_linear_cross_entropy import (
    _infer_weight_layout,
    tiled_linear_cross_entropy,
)

REPO_ROOT = Path(__file__).resolve().parent.parent


def test_package_export_is_lazy_callable():
    result = subprocess.run(
        [sys.executable, "-c",
         "import sys; from turbo_dllm_amd import tiled_linear_cross_entropy; "
         "print(callable(tiled_linear_cross_entropy), 'torch' in sys.modules)"],
        check=True, capture_output=True, text=True, cwd=REPO_ROOT)
    assert result.stdout.strip() == "True False"


@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_matches_dense_loss_and_grads(reduction):
    torch.manual_seed(0)
    hidden = torch.randn(2, 5, 7, requires_grad=True)
    weight = torch.randn(13, 7, requires_grad=True)
    bias = torch.randn(13, requires_grad=True)
    labels = torch.randint(0, 13, (2, 5))
    labels[0, 1] = -100
    loss = tiled_linear_cross_entropy(hidden, weight, labels, bias=bias, vocab_block_size=4,
                                      reduction=reduction)
    ref = oracle.dense_linear_ce(hidden.detach(), weight.detach(), labels, bias=bias.detach(),
                                 reduction=reduction)
    assert loss.dtype == torch.float32
    torch.testing.assert_close(loss, ref.float(), atol=2e-5, rtol=2e-5)
    grad = torch.randn_like(loss) if reduction == "none" else None
    loss.backward(grad)
    dh, dw, db = oracle.dense_linear_ce_grads(hidden.detach(), weight.detach(), labels, grad,
                                              bias=bias.detach(), reduction=reduction)
    torch.testing.assert_close(hidden.grad, dh.float(), atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(weight.grad, dw.float(), atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(bias.grad, db.float(), atol=3e-5, rtol=3e-5)


def test_dim_first_weight():
    torch.manual_seed(1)
    hidden = torch.randn(3, 4, requires_grad=True)
    weight = torch.randn(4, 9, requires_grad=True)
    labels = torch.tensor([0, 5, 8])
    loss = tiled_linear_cross_entropy(hidden, weight, labels, vocab_block_size=3,
                                      reduction="none", weight_layout="dim_first")
    ref = F.cross_entropy(hidden.detach() @ weight.detach(), labels, reduction="none")
    torch.testing.assert_close(loss, ref, atol=2e-5, rtol=2e-5)
    loss.sum().backward()
    _, dw, _ = oracle.dense_linear_ce_grads(hidden.detach(), weight.detach(), labels,
                                            reduction="sum", weight_dim_first=True)
    assert weight.grad.shape == weight.shape
    torch.testing.assert_close(weight.grad, dw.float(), atol=3e-5, rtol=3e-5)


def test_excludes_mask_token():
    torch.manual_seed(2)
    hidden = torch.randn(2, 3, 5, requires_grad=True)
    weight = torch.randn(11, 5, requires_grad=True)
    labels = torch.randint(0, 10, (2, 3))
    loss = tiled_linear_cross_entropy(hidden, weight, labels, vocab_block_size=4,
                                      reduction="mean", exclude_index=10)
    logits = hidden.detach().reshape(-1, 5) @ weight.detach().t()
    logits[:, 10] = -float("inf")
    torch.testing.assert_close(loss, F.cross_entropy(logits, labels.reshape(-1)), atol=2e-5,
                               rtol=2e-5)
    loss.backward()
    assert torch.count_nonzero(weight.grad[10]) == 0


def test_non_contiguous_inputs():
    torch.manual_seed(3)
    hidden = torch.randn(2, 8, 6)[:, ::2, :].requires_grad_(True)
    labels = torch.randint(0, 17, (2, 8))[:, ::2]
    weight = torch.randn(17, 6, requires_grad=True)
    assert not hidden.is_contiguous() and not labels.is_contiguous()
    loss = tiled_linear_cross_entropy(hidden, weight, labels, vocab_block_size=5)
    ref = oracle.dense_linear_ce(hidden.detach(), weight.detach(), labels)
    torch.testing.assert_close(loss, ref.float(), atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("tile", [1, 5, 7, 64])
def test_vocab_tile_sizes_are_equivalent(tile):
    torch.manual_seed(31)
    hidden = torch.randn(3, 5, 9, requires_grad=True)
    weight = torch.randn(23, 9, requires_grad=True)
    bias = torch.randn(23, requires_grad=True)
    labels = torch.randint(0, 22, (3, 5))
    labels[0, 0] = -100
    labels[2, 4] = -100
    grad_out = torch.randn(3, 5)
    loss = tiled_linear_cross_entropy(hidden, weight, labels, bias=bias, vocab_block_size=tile,
                                      reduction="none", exclude_index=22)
    ref = oracle.dense_linear_ce(hidden.detach(), weight.detach(), labels, bias=bias.detach(),
                                 reduction="none", exclude_index=22)
    torch.testing.assert_close(loss, ref.float(), atol=2e-5, rtol=2e-5)
    loss.backward(grad_out)
    dh, dw, db = oracle.dense_linear_ce_grads(hidden.detach(), weight.detach(), labels, grad_out,
                                              bias=bias.detach(), reduction="none",
                                              exclude_index=22)
    torch.testing.assert_close(hidden.grad, dh.float(), atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(weight.grad, dw.float(), atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(bias.grad, db.float(), atol=3e-5, rtol=3e-5)


def test_bfloat16_inputs_float32_compute():
    torch.manual_seed(4)
    hidden = torch.randn(2, 4, 8, dtype=torch.bfloat16)
    weight = torch.randn(19, 8, dtype=torch.bfloat16)
    labels = torch.randint(0, 19, (2, 4))
    loss = tiled_linear_cross_entropy(hidden, weight, labels, vocab_block_size=7,
                                      dtype=torch.float32)
    ref = oracle.dense_linear_ce(hidden, weight, labels)
    torch.testing.assert_close(loss, ref.float(), atol=3e-2, rtol=3e-2)


def test_large_vocab_smoke_backward():
    torch.manual_seed(5)
    hidden = torch.randn(2, 16, 16, requires_grad=True)
    weight = torch.randn(32768, 16, requires_grad=True)
    labels = torch.randint(0, 32768, (2, 16))
    loss = tiled_linear_cross_entropy(hidden, weight, labels, vocab_block_size=1024)
    assert torch.isfinite(loss)
    loss.backward()
    assert hidden.grad.shape == hidden.shape and weight.grad.shape == weight.shape


def test_subs_masked_token_loss_equivalence():
    # test_tiled_linear_cross_entropy.py:408-453: CE on masked positions with the
    # mask token excluded equals the SUBS log-probability form
    torch.manual_seed(6)
    batch, seq_len, hidden_dim, vocab = 2, 6, 7, 23
    mask_index = vocab - 1
    hidden = torch.randn(batch, seq_len, hidden_dim)
    weight = torch.randn(vocab, hidden_dim)
    bias = torch.randn(vocab)
    x0 = torch.randint(0, vocab - 1, (batch, seq_len))
    xt = x0.clone()
    xt[0, 1] = xt[0, 4] = xt[1, 2] = mask_index
    loss_scale = -torch.rand(batch, seq_len)
    logits = hidden @ weight.t() + bias
    logits[:, :, mask_index] = -float("inf")
    log_probs = logits - torch.logsumexp(logits, dim=-1, keepdim=True)
    unmasked = xt != mask_index
    log_probs[unmasked] = -float("inf")
    log_probs[unmasked, xt[unmasked]] = 0
    ref = loss_scale * torch.gather(log_probs, -1, x0[:, :, None]).squeeze(-1)
    labels = torch.where(xt == mask_index, x0, torch.full_like(x0, -100))
    ce = tiled_linear_cross_entropy(hidden, weight, labels, bias=bias, vocab_block_size=5,
                                    reduction="none", exclude_index=mask_index)
    torch.testing.assert_close(-loss_scale * ce, ref, atol=2e-5, rtol=2e-5)


def test_softcap_then_exclusion_is_true_removal():
    # native-path semantics: the excluded column leaves the softmax also under a cap
    torch.manual_seed(7)
    hidden = torch.randn(6, 16) * 3
    weight = torch.randn(37, 16)
    labels = torch.randint(5, 37, (6,))
    got = tiled_linear_cross_entropy(hidden, weight, labels, reduction="none", exclude_index=4,
                                     logit_softcap=5.0, vocab_block_size=8)
    logits = torch.tanh(hidden @ weight.t() / 5.0) * 5.0
    logits[:, 4] = -float("inf")
    torch.testing.assert_close(got, F.cross_entropy(logits, labels, reduction="none"), atol=2e-5,
                               rtol=2e-5)


def test_error_behaviour():
    hidden = torch.randn(4, 6)
    weight = torch.randn(9, 6)
    labels = torch.tensor([0, 1, 2, 3])
    with pytest.raises(ValueError, match="must match hidden prefix"):
        tiled_linear_cross_entropy(hidden, weight, labels[:3])
    with pytest.raises(ValueError, match="labels must be in"):
        tiled_linear_cross_entropy(hidden, weight, torch.tensor([0, 1, 2, 9]))
    with pytest.raises(ValueError, match="may not equal exclude_index"):
        tiled_linear_cross_entropy(hidden, weight, labels, exclude_index=2)
    with pytest.raises(ValueError, match="reduction must be"):
        tiled_linear_cross_entropy(hidden, weight, labels, reduction="avg")
    with pytest.raises(ValueError, match="Unsupported dtype"):
        tiled_linear_cross_entropy(hidden, weight, labels, dtype="int8")
    with pytest.raises(ValueError, match="bias must have shape"):
        tiled_linear_cross_entropy(hidden, weight, labels, bias=torch.zeros(8))
    with pytest.raises(ValueError, match="Could not infer"):
        tiled_linear_cross_entropy(hidden, torch.randn(9, 5), labels)
    with pytest.raises(ValueError, match="weight_layout must be"):
        _infer_weight_layout(6, weight, "row")
    assert _infer_weight_layout(6, weight, "auto") is False
    assert _infer_weight_layout(6, weight.t(), "auto") is True
    assert _infer_weight_layout(6, torch.randn(6, 6), "auto") is False  # last dim wins
    # all rows ignored: mean is 0/0 = nan, as the reference (no clamp), sum is 0
    ignored = torch.full((4,), -100)
    assert torch.isnan(tiled_linear_cross_entropy(hidden, weight, ignored))
    assert float(tiled_linear_cross_entropy(hidden, weight, ignored, reduction="sum")) == 0.0


def test_compaction_and_loss_wrapper_on_host():
    from turbo_dllm_amd.compaction import compact_valid_loss_rows
    from turbo_dllm_amd.layers import VocabParallelLinear
    from turbo_dllm_amd.loss import masked_token_loss

    torch.manual_seed(9)
    hidden = torch.randn(2, 6, 8, requires_grad=True)
    labels = torch.randint(0, 20, (2, 6))
    labels[0, ::2] = -100
    weights = torch.rand(2, 6)
    rows, targets, w = compact_valid_loss_rows(hidden, labels, weights, ignore_index=-100)
    keep = labels.reshape(-1) != -100
    torch.testing.assert_close(rows, hidden.reshape(-1, 8)[keep])
    assert torch.equal(targets, labels.reshape(-1)[keep])
    torch.testing.assert_close(w, weights.reshape(-1)[keep])
    # all valid: returned as passed, only the weights flattened
    full = torch.randint(0, 20, (2, 6))
    rows, targets, w = compact_valid_loss_rows(hidden, full, weights, ignore_index=-100)
    assert rows is hidden and targets is full and w.shape == (12,)

    head = VocabParallelLinear(8, 20, bias=True)
    loss = masked_token_loss(hidden, labels, weights, head, valid_token_count=9.0,
                             mask_token_id=19, output_multiplier=0.5, loss_scale=2.0)
    logits = F.linear(hidden.detach().reshape(-1, 8) * 0.5, head.weight, head.bias)
    logits[:, 19] = -float("inf")
    labels19 = labels.reshape(-1)
    ce = F.cross_entropy(logits, labels19, reduction="none", ignore_index=-100)
    ref = (ce * weights.reshape(-1)).sum() / 9.0 * 2.0
    torch.testing.assert_close(loss, ref, atol=2e-5, rtol=2e-5)
    loss.backward()
    assert hidden.grad is not None and head.weight.grad is not None
    # no supervised row: exact zero that still reaches every parameter
    empty = masked_token_loss(hidden, torch.full((2, 6), -100), weights, head,
                              valid_token_count=1.0)
    assert float(empty.detach()) == 0.0
    empty.backward()
    with pytest.raises(NotImplementedError):
        VocabParallelLinear(8, 20, tensor_parallel_size=2)


def test_native_token_cross_entropy_on_host_and_compaction_modes():
    from turbo_dllm_amd.loss import native_token_cross_entropy
    from turbo_dllm_amd.tiled_linear_cross_entropy import (COMPACTION_MODES, compaction_mode,
                                                           get_compaction_mode,
                                                           set_compaction_mode)

    torch.manual_seed(8)
    hidden = torch.randn(7, 8, requires_grad=True)
    labels = torch.randint(0, 20, (7,))
    head = torch.nn.Linear(8, 20, bias=True)
    losses = native_token_cross_entropy(hidden, labels, head, output_multiplier=0.5,
                                        logit_softcap=6.0)
    logits = F.linear(hidden.detach() * 0.5, head.weight, head.bias)
    logits = torch.tanh(logits / 6.0) * 6.0
    ref = F.cross_entropy(logits, labels, reduction="none")
    assert losses.shape == labels.shape and losses.dtype == torch.float32
    torch.testing.assert_close(losses, ref, atol=2e-5, rtol=2e-5)
    losses.sum().backward()
    assert hidden.grad is not None and head.weight.grad is not None

    # the compaction mode is a context-local setting with a scoped form
    assert COMPACTION_MODES == ("sync", "device", "none") and get_compaction_mode() == "sync"
    with compaction_mode("device"):
        assert get_compaction_mode() == "device"
        with compaction_mode("none"):
            assert get_compaction_mode() == "none"
        assert get_compaction_mode() == "device"
    assert get_compaction_mode() == "sync"
    with pytest.raises(ValueError):
        set_compaction_mode("lazy")
    assert get_compaction_mode() == "sync"


def test_options_are_local_to_the_calling_thread():
    """Two trainers in one process can choose different compaction modes and
    panel budgets: a setting made in one thread is invisible in another."""
    import threading

    from turbo_dllm_amd import options

    seen = {}
    ready, release = threading.Event(), threading.Event()

    def other():
        seen["start"] = (options.get_compaction_mode(), options.get_panel_bytes())
        with options.compaction_mode("none"), options.panel_budget(1 << 20):
            ready.set()
            release.wait(10)
            seen["inside"] = (options.get_compaction_mode(), options.get_panel_bytes())

    with options.compaction_mode("device"), options.panel_budget(1 << 28):
        thread = threading.Thread(target=other)
        thread.start()
        assert ready.wait(10)
        # the other thread's choices did not leak into this one
        assert options.get_compaction_mode() == "device" and options.get_panel_bytes() == 1 << 28
        release.set()
        thread.join(10)
    assert seen["start"] == ("sync", 0)            # a new thread starts from the defaults
    assert seen["inside"] == ("none", 1 << 20)
    assert options.get_compaction_mode() == "sync" and options.get_panel_bytes() == 0
    assert options.resolve_compaction(None) == "sync"
    assert options.resolve_compaction("device") == "device"
    with pytest.raises(ValueError):
        options.resolve_compaction("lazy")
    with pytest.raises(ValueError):
        with options.panel_budget(-1):
            pass
    old = options.set_panel_bytes(4096)
    assert old == 0 and options.get_panel_bytes() == 4096
    options.set_panel_bytes(old)


def test_gradient_mode_option_and_host_tensors():
    """The gradient mode is a context-local option like the others; host tensors
    never take the library's forward-with-gradients path, whatever the mode."""
    import threading

    from turbo_dllm_amd import chunked_linear_ce_native as native
    from turbo_dllm_amd import options
    from turbo_dllm_amd.tiled_linear_cross_entropy import tiled_linear_cross_entropy

    assert options.GRADIENT_MODES == ("forward", "recompute")
    assert options.get_gradient_mode() == "forward"
    seen = {}
    with options.gradient_mode("recompute"):
        thread = threading.Thread(target=lambda: seen.update(mode=options.get_gradient_mode()))
        thread.start()
        thread.join(10)
        assert options.get_gradient_mode() == "recompute"
    assert seen["mode"] == "forward" and options.get_gradient_mode() == "forward"
    with pytest.raises(ValueError):
        options.set_gradient_mode("lazy")
    old = options.set_gradient_mode("recompute")
    assert old == "forward"
    options.set_gradient_mode(old)

    gen = torch.Generator().manual_seed(0)
    hidden = torch.randn(6, 64, generator=gen).bfloat16()
    weight = torch.randn(128, 64, generator=gen).bfloat16()
    labels = torch.randint(0, 128, (6,), generator=gen)
    assert not native.fused_gradients_supported(hidden, weight, None, False)   # host tensors
    results = []
    for mode in options.GRADIENT_MODES:
        x = hidden.clone().requires_grad_(True)
        with options.gradient_mode(mode):
            loss = tiled_linear_cross_entropy(x, weight, labels, dtype=torch.float32,
                                              weight_layout="vocab_first")
            loss.backward()
        results.append((loss.detach(), x.grad))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])


def test_verify_dflash_symbols():
    """Start-up check of the DFlash executor (reference shim,
    chunked_linear_ce_native.py:353-363): unknown kinds raise ValueError, known
    ones resolve the library and the entry points that loss needs."""
    from turbo_dllm_amd import _lib
    from turbo_dllm_amd import chunked_linear_ce_native as native

    for kind in ("paper_ce", "speculators_kl", "dflash", "dpace",
                 "dpace-cumulative-confidence-only", "dpace-continuation-value-only"):
        native.verify_dflash_symbols(loss_kind=kind)
    with pytest.raises(ValueError, match="unsupported DFlash loss 'kl'"):
        native.verify_dflash_symbols(loss_kind="kl")
    with pytest.raises(TypeError):
        native.verify_dflash_symbols("paper_ce")        # keyword-only, as in the reference
    # a library without the entry points fails the check, not the first training step
    class Stub:
        pass
    real = _lib.library
    try:
        _lib.library = lambda: Stub()
        with pytest.raises(_lib.NativeLibraryMissing, match="tlce_kl_workspace_bytes"):
            native.verify_dflash_symbols(loss_kind="speculators_kl")
    finally:
        _lib.library = real
