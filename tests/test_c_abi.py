"""The C-ABI library loads, exports exactly what include/tlce.h declares, and
its host-side planning logic behaves (no compute calls: no GPU needed)."""

import ctypes
import re
from pathlib import Path

import pytest

from turbo_dllm_amd import _lib

REPO_ROOT = Path(__file__).resolve().parent.parent
HEADER = REPO_ROOT / "include" / "tlce.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    names = re.findall(r"\b(tlce_[a-z_0-9]+)\s*\(", text)
    return sorted(set(names))


def test_header_and_binding_declare_the_same_entry_points():
    assert declared_functions() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = _lib.library()
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert lib.tlce_version() == 1
    assert _lib.last_error() == ""


def test_argument_counts_match_header():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        match = re.search(rf"\b{name}\s*\(([^)]*)\)", text)
        assert match, name
        params = match.group(1).strip()
        count = 0 if params in ("", "void") else len(params.split(","))
        assert count == len(argtypes), (name, count, len(argtypes))


def test_workspace_sizes_and_plan():
    lib = _lib.library()
    assert lib.tlce_compact_workspace_bytes(0) >= 4
    assert lib.tlce_compact_workspace_bytes(32768) >= 32 * 4
    assert lib.tlce_compact_workspace_bytes(-1) == -1
    # headline shape: MFMA engine, 256 tiles, vocabulary panels bounded by 1 GiB
    plan = _lib.query_plan(32768, 4096, 151936, _lib.DTYPE_BF16, True)
    assert plan["engine"] == "mfma_direct" and plan["tile"] == 256
    assert plan["forward_vocab_splits"] == 8
    assert plan["panel_columns"] % 256 == 0
    # one panel orientation only: grad_weight reads the panel K-major, in place
    assert plan["panel_columns"] * 32768 * 2 <= (1 << 30)
    assert plan["n_panels"] * plan["panel_columns"] >= 151936
    assert plan["grad_hidden_k_splits"] == 1
    fwd = lib.tlce_forward_workspace_bytes(32768, 4096, 151936, _lib.DTYPE_BF16)
    assert fwd == 2 * 8 * 32768 * 4  # (max, sum) float32 partials only: the forward stores no logits
    # the backward stages rounded logit GRADIENTS in one bounded vocabulary panel (1 GiB by
    # default: 16384 of the 151936 columns, 5.4 % of the float32 logits matrix the reference
    # blocks through); it is a [rows, panel] buffer, not "no buffer"
    bwd = lib.tlce_backward_workspace_bytes(32768, 4096, 151936, _lib.DTYPE_BF16, 1, 0, 0)
    logits_bytes = 32768 * 151936 * 4
    panel_bytes = plan["panel_columns"] * 32768 * 2
    assert panel_bytes == 1 << 30 and panel_bytes * 18 < logits_bytes
    assert bwd < logits_bytes // 4
    # the device-side row count needs room for whatever plan a smaller count selects
    dyn = lib.tlce_masked_loss_forward_workspace_bytes(32768, 4096, 151936, _lib.DTYPE_BF16, 1)
    assert dyn == 2 * 1024 * 256 * 4 + 32768 * 4
    assert lib.tlce_masked_loss_forward_workspace_bytes(32768, 4096, 151936, _lib.DTYPE_BF16, 0) \
        == fwd + 32768 * 4
    frozen = lib.tlce_backward_workspace_bytes(32768, 4096, 151936, _lib.DTYPE_BF16, 0, 0, 0)
    assert frozen <= bwd
    # float32 grad_hidden accumulators + one bf16 panel + per-row scales, nothing else
    assert bwd == 32768 * 4096 * 4 + plan["panel_columns"] * 32768 * 2 + 32768 * 4
    # a vocabulary that is not a multiple of 64 falls back to transposed operand copies
    assert lib.tlce_backward_workspace_bytes(32768, 4096, 151937, _lib.DTYPE_BF16, 1, 0, 0) > bwd
    # few loss rows: the grad-hidden contraction splits K to fill the GPU
    small = _lib.query_plan(1750, 4096, 151936, _lib.DTYPE_BF16, True)
    assert small["n_panels"] <= 2 and small["grad_hidden_k_splits"] > 1
    # float32 inputs and odd hidden sizes take the generic engine
    assert _lib.query_plan(21, 33, 4097, _lib.DTYPE_F32, True)["engine"] == "generic"
    assert _lib.query_plan(21, 33, 4097, _lib.DTYPE_BF16, True)["engine"] == "generic"
    assert _lib.query_plan(31, 96, 1025, _lib.DTYPE_BF16, True)["engine"] == "mfma"  # K tail
    assert _lib.query_plan(64, 128, 300, _lib.DTYPE_BF16, True)["engine"] == "mfma_direct"
    # a smaller panel budget means more panels
    tight = _lib.query_plan(32768, 4096, 151936, _lib.DTYPE_BF16, True, 1 << 28)
    assert tight["n_panels"] > plan["n_panels"]


def test_bad_arguments_report_errors_without_a_gpu():
    lib = _lib.library()
    rc = lib.tlce_query_plan(1, 0, 5, _lib.DTYPE_BF16, 1, 0, None, None, None, None, None, None)
    assert rc != 0 and "bad shape" in _lib.last_error()
    with pytest.raises(RuntimeError, match="bad shape"):
        _lib.check(rc, "tlce_query_plan")
    assert lib.tlce_forward_workspace_bytes(-1, 8, 8, _lib.DTYPE_BF16) == -1


def test_masked_loss_entry_points_validate_before_touching_a_gpu():
    lib = _lib.library()
    fake = 4096          # aligned, never dereferenced: validation fails first
    common = (fake, fake, None, fake, None, None, None, 8, 8, 64, 100, _lib.DTYPE_BF16)
    # the logit multiplier must be positive (the kernels keep maxima of unscaled dot products)
    rc = lib.tlce_masked_loss_forward(*common, -100, -1, 0.0, -0.5, None, fake, fake, fake,
                                      fake, 1 << 20, None)
    assert rc != 0 and "multiplier must be positive" in _lib.last_error()
    rc = lib.tlce_masked_loss_backward(fake, fake, None, fake, None, None, None, fake, None, fake,
                                       8, 8, 64, 100, _lib.DTYPE_BF16, _lib.REDUCTION_SUM,
                                       -100, -1, 0.0, 0.0, fake, None, None, 0, fake, 1 << 30, None)
    assert rc != 0 and "multiplier must be positive" in _lib.last_error()
    # neither per-token losses nor the weighted sum asked for
    rc = lib.tlce_masked_loss_forward(*common, -100, -1, 0.0, 1.0, None, fake, fake, None,
                                      fake, 1 << 20, None)
    assert rc != 0 and "neither" in _lib.last_error()
    # gather: the weights go in and out together
    rc = lib.tlce_gather_loss_rows(fake, fake, fake, fake, fake, 8, 64, 128, -100, fake, fake,
                                   None, None)
    assert rc != 0 and "weights" in _lib.last_error()
    assert lib.tlce_masked_loss_forward_workspace_bytes(-1, 8, 8, _lib.DTYPE_BF16, 0) == -1


def test_dim_first_entry_points_validate_before_touching_a_gpu():
    lib = _lib.library()
    assert lib.tlce_dim_first_supported(4096, 151936, _lib.DTYPE_BF16) == 1
    assert lib.tlce_dim_first_supported(4096, 151936, _lib.DTYPE_F32) == 0     # float32 inputs
    assert lib.tlce_dim_first_supported(4096, 151937, _lib.DTYPE_BF16) == 0    # partial K slab
    assert lib.tlce_dim_first_supported(72, 1024, _lib.DTYPE_BF16) == 0        # staged engine
    assert lib.tlce_dim_first_supported(0, 64, _lib.DTYPE_BF16) == 0
    fake = 4096          # aligned, never dereferenced: validation fails first
    rc = lib.tlce_forward_dim_first(fake, fake, None, fake, None, 8, 8, 64, 100, _lib.DTYPE_BF16,
                                    -100, -1, 0.0, fake, fake, fake, fake, 1 << 20, None)
    assert rc != 0 and "read in place only" in _lib.last_error()
    rc = lib.tlce_backward_dim_first(fake, fake, None, fake, None, fake, fake, fake, 8, 8, 64, 100,
                                     _lib.DTYPE_F32, _lib.REDUCTION_SUM, -100, -1, 0.0, fake,
                                     fake, None, 0, fake, 1 << 30, None)
    assert rc != 0 and "read in place only" in _lib.last_error()


def test_fused_gradient_entry_points_validate_before_touching_a_gpu():
    lib = _lib.library()
    assert lib.tlce_fused_gradients_supported(4096, 151936, _lib.DTYPE_BF16) == 1
    assert lib.tlce_fused_gradients_supported(4096, 151936, _lib.DTYPE_F16) == 0    # bf16 only
    assert lib.tlce_fused_gradients_supported(4096, 151936, _lib.DTYPE_F32) == 0
    assert lib.tlce_fused_gradients_supported(4096, 151937, _lib.DTYPE_BF16) == 0
    assert lib.tlce_fused_gradients_supported(72, 1024, _lib.DTYPE_BF16) == 0
    assert lib.tlce_forward_with_gradients_workspace_bytes(8, 72, 1024, _lib.DTYPE_BF16, 1, 0) == -1
    fake = 4096          # aligned, never dereferenced: validation fails first

    def forward(h=64, v=128, dtype=_lib.DTYPE_BF16, multiplier=1.0, ws_bytes=1 << 30, n_out=8,
                row_idx=None, row_count=None):
        return lib.tlce_forward_with_gradients(
            fake, fake, fake, row_idx, None, row_count, 8, n_out, h, v, dtype, -100, -1, 0.0,
            multiplier, fake, fake, fake, fake, fake, 0, fake, ws_bytes, None)

    assert forward(h=72) != 0 and "multiples of 64" in _lib.last_error()
    assert forward(dtype=_lib.DTYPE_F32) != 0 and "multiples of 64" in _lib.last_error()
    assert forward(multiplier=0.0) != 0 and "multiplier must be positive" in _lib.last_error()
    assert forward(ws_bytes=16) != 0 and "workspace too small" in _lib.last_error()
    assert forward(n_out=4) != 0 and "n_out" in _lib.last_error()
    assert forward(n_out=16) != 0 and "without row_idx" in _lib.last_error()
    assert forward(row_count=fake) != 0 and "needs row_idx" in _lib.last_error()
    # one upstream gradient per row: grad_weight cannot be finished from a float32 sum
    rc = lib.tlce_apply_grad_output(fake, fake, None, None, fake, fake, 8, 8, 64, 128,
                                    _lib.DTYPE_BF16, _lib.REDUCTION_NONE, fake, fake, None)
    assert rc != 0 and "has to wait" in _lib.last_error()
    rc = lib.tlce_apply_grad_output(fake, None, None, None, fake, fake, 8, 8, 64, 128,
                                    _lib.DTYPE_BF16, 7, fake, None, None)
    assert rc != 0 and "unknown reduction" in _lib.last_error()
    rc = lib.tlce_apply_grad_output(fake, None, None, None, fake, fake, 8, 8, 64, 128,
                                    _lib.DTYPE_BF16, _lib.REDUCTION_SUM, fake, fake, None)
    assert rc != 0 and "go together" in _lib.last_error()
    rc = lib.tlce_apply_grad_output(fake, fake, None, None, fake, None, 8, 8, 64, 128,
                                    _lib.DTYPE_BF16, _lib.REDUCTION_MEAN, fake, fake, None)
    assert rc != 0 and "valid_count" in _lib.last_error()


def test_postponed_weight_gradient_entry_validates_before_touching_a_gpu():
    import torch

    from turbo_dllm_amd import chunked_linear_ce_native as native
    from turbo_dllm_amd import options

    lib = _lib.library()
    fake = 4096

    def call(m=8, h=64, v=128, dtype=_lib.DTYPE_BF16, reduction=_lib.REDUCTION_SUM,
             panel=0, ws_bytes=1 << 30, valid=fake):
        return lib.tlce_grad_weight_from_panel(fake, None, None, fake, valid, m, h, v, dtype,
                                               reduction, fake, panel, fake, ws_bytes, None)

    assert call(h=72) != 0 and "multiples of 64" in _lib.last_error()
    assert call(reduction=7) != 0 and "unknown reduction" in _lib.last_error()
    assert call(reduction=_lib.REDUCTION_MEAN, valid=None) != 0 and "valid_count" in _lib.last_error()
    assert call(ws_bytes=16) != 0 and "workspace too small" in _lib.last_error()
    # 600 rows over a 128-word vocabulary with a one-tile panel: three blocks of rows
    assert call(m=600, panel=1) != 0 and "blocks of rows" in _lib.last_error()
    # whether the contraction can wait follows the plan under the budget in force
    assert native.weight_grad_can_wait(8298, 4096, 151936, torch.bfloat16)
    assert not native.weight_grad_can_wait(32768, 4096, 151936, torch.bfloat16)
    assert not native.weight_grad_can_wait(8298, 4096, 151936, torch.float16)
    with options.panel_budget(1 << 30):
        assert not native.weight_grad_can_wait(8298, 4096, 151936, torch.bfloat16)


def test_fused_plan_blocks():
    # the benchmark's shape: 2.5 GiB hold 34 token tiles over 594 vocabulary tiles; four
    # balanced blocks of 32 tiles (whole rounds of 256 workgroups for grad_hidden)
    plan = _lib.query_fused_plan(32768, 4096, 151936, _lib.DTYPE_BF16)
    assert plan == {"block_rows": 8192, "n_blocks": 4, "grad_hidden_k_splits": 1}
    # a 1 GiB panel: 13 tiles fit, ten balanced blocks
    plan = _lib.query_fused_plan(32768, 4096, 151936, _lib.DTYPE_BF16, 1 << 30)
    assert plan["block_rows"] == 13 * 256 and plan["n_blocks"] == 10
    # everything in one block when it fits; the K split then fills the chip
    plan = _lib.query_fused_plan(1610, 4096, 151936, _lib.DTYPE_BF16)
    assert plan["n_blocks"] == 1 and plan["block_rows"] == 1792
    assert plan["grad_hidden_k_splits"] > 1
    # a budget below one tile still makes progress, one token tile at a time
    plan = _lib.query_fused_plan(1000, 256, 5120, _lib.DTYPE_BF16, 1)
    assert plan["block_rows"] == 256 and plan["n_blocks"] == 4
    bytes_needed = _lib.library().tlce_forward_with_gradients_workspace_bytes(
        32768, 4096, 151936, _lib.DTYPE_BF16, 1, 0)
    panel = 8192 * 152064 * 2
    assert panel < bytes_needed < panel + (1 << 30)
