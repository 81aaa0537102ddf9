"""Frozen-head CE with exact top-k: argument checks and the dense path on the
CPU, the device path against the float64 oracle."""

import pytest
import torch

import linear_ce_oracle as oracle
from turbo_dllm_amd.dflash_linear_topk import frozen_linear_ce_topk


def test_argument_checks():
    h, w, y = torch.randn(4, 8), torch.randn(11, 8), torch.randint(0, 11, (4,))
    with pytest.raises(ValueError, match=r"expects \[N,D\], \[V,D\], and \[N\]"):
        frozen_linear_ce_topk(h, w, y[None], top_k=2)
    with pytest.raises(ValueError, match="dimensions are incompatible"):
        frozen_linear_ce_topk(h, torch.randn(11, 7), y, top_k=2)
    with pytest.raises(ValueError, match="frozen weight"):
        frozen_linear_ce_topk(h, w.clone().requires_grad_(True), y, top_k=2)
    with pytest.raises(ValueError, match="vocabulary range"):
        frozen_linear_ce_topk(h, w, y, top_k=12)
    with pytest.raises(ValueError, match="outside the vocabulary"):
        frozen_linear_ce_topk(h, w, torch.full((4,), 11), top_k=2)
    with pytest.raises(ValueError, match="must be positive"):
        frozen_linear_ce_topk(h, w, y, top_k=2, logit_softcap=0.0)


@pytest.mark.parametrize("softcap,mult", [(None, 1.0), (3.0, 0.5)])
def test_dense_path_matches_oracle(softcap, mult):
    torch.manual_seed(5)
    n, h, v, k = 9, 6, 23, 5
    hidden = torch.randn(n, h, requires_grad=True)
    weight = torch.randn(v, h)
    labels = torch.randint(0, v, (n,))
    loss, prob, vals, ids = frozen_linear_ce_topk(hidden, weight, labels, top_k=k,
                                                  output_multiplier=mult, logit_softcap=softcap)
    gl, gp, gv = torch.randn(n), torch.randn(n), torch.randn(n, k)
    ((gl * loss).sum() + (gp * prob).sum() + (gv * vals).sum()).backward()
    r_loss, r_prob, r_vals, r_ids, _ = oracle.dense_ce_topk(
        hidden.detach(), weight, labels, k, output_multiplier=mult, logit_softcap=softcap)
    torch.testing.assert_close(loss.double(), r_loss, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(prob.double(), r_prob, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(vals.double(), r_vals, rtol=1e-5, atol=1e-5)
    assert torch.equal(ids, r_ids)
    r_grad = oracle.dense_ce_topk_grad(hidden.detach(), weight, labels, ids, gl, gp, gv,
                                       output_multiplier=mult, logit_softcap=softcap)
    torch.testing.assert_close(hidden.grad.double(), r_grad, rtol=1e-4, atol=1e-5)


GPU_CASES = [
    # name, dtype, N, H, V, k, softcap, multiplier, weight std, panel bytes
    ("bf16_staged_h72", torch.bfloat16, 61, 72, 1025, 4, None, 1.0, 0.3, 0),
    ("bf16_direct", torch.bfloat16, 300, 256, 2304, 8, None, 1.0, 0.1, 0),
    ("bf16_direct_softcap_mult", torch.bfloat16, 129, 128, 1536, 16, 5.0, 0.6, 0.3, 0),
    ("f16_three_panels_k1", torch.float16, 520, 64, 1024, 1, None, 1.0, 0.3, 768 * 512 * 4),
    ("bf16_wide_chunks_k33", torch.bfloat16, 40, 64, 40000, 33, None, 2.0, 0.2, 0),
    # k = 256: far more logits reach the first threshold than the gather holds -> selection rounds
    ("bf16_k256_rounds", torch.bfloat16, 33, 64, 20000, 256, None, 1.0, 0.3, 0),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", GPU_CASES, ids=[c[0] for c in GPU_CASES])
def test_device_path_matches_oracle(gpu_device, case, set_panel_budget):
    name, dtype, n, h, v, k, softcap, mult, std, panel_bytes = case
    print("[case]", name, flush=True)
    if panel_bytes:
        set_panel_budget(panel_bytes)
    gen = torch.Generator().manual_seed(len(name) + k)
    hidden = torch.randn(n, h, generator=gen).to(dtype)
    weight = (torch.randn(v, h, generator=gen) * std).to(dtype)
    labels = torch.randint(0, v, (n,), generator=gen)
    gl, gp, gv = (torch.randn(n, generator=gen), torch.randn(n, generator=gen),
                  torch.randn(n, k, generator=gen))
    x = hidden.to(gpu_device).requires_grad_(True)
    loss, prob, vals, ids = frozen_linear_ce_topk(x, weight.to(gpu_device), labels.to(gpu_device),
                                                  top_k=k, output_multiplier=mult,
                                                  logit_softcap=softcap)
    ((gl.to(gpu_device) * loss).sum() + (gp.to(gpu_device) * prob).sum()
     + (gv.to(gpu_device) * vals).sum()).backward()
    torch.cuda.synchronize()
    r_loss, r_prob, r_vals, r_ids, _ = oracle.dense_ce_topk(
        hidden, weight, labels, k, output_multiplier=mult, logit_softcap=softcap)
    z = oracle._topk_logits(hidden, weight, mult, softcap, torch.float64)[0]
    loss, prob, vals, ids = (t.detach().cpu() for t in (loss, prob, vals, ids))
    torch.testing.assert_close(loss.double(), r_loss, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(prob.double(), r_prob, rtol=2e-3, atol=1e-4)
    # the values are the row's k largest logits in descending order, and the ids name them;
    # ids may differ from the oracle's only where float32 rounding reorders near-equal logits
    torch.testing.assert_close(vals.double(), r_vals, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(z.gather(1, ids), vals.double(), rtol=1e-3, atol=1e-3)
    assert bool((vals[:, :-1] >= vals[:, 1:]).all()) if k > 1 else True
    assert ids.dtype == torch.long and bool(((ids >= 0) & (ids < v)).all())
    assert all(len(set(row)) == k for row in ids.tolist())
    agree = float((ids == r_ids).double().mean())
    print("[case] ids agreeing with the oracle", agree, flush=True)
    assert agree > 0.97
    r_grad = oracle.dense_ce_topk_grad(hidden, weight, labels, ids, gl, gp, gv,
                                       output_multiplier=mult, logit_softcap=softcap)
    err = oracle.relative_max_error(x.grad.cpu(), r_grad)
    print("[case] grad rel max err", f"{err:.2e}", flush=True)
    assert err <= 2e-2


@pytest.mark.gpu
def test_only_loss_gradient_matches_cross_entropy_backward(gpu_device):
    """With gradients for the loss alone the result equals the frozen-weight
    cross-entropy backward of the main path."""
    from turbo_dllm_amd.tiled_linear_cross_entropy import tiled_linear_cross_entropy
    gen = torch.Generator().manual_seed(3)
    n, h, v = 260, 128, 2048
    hidden = torch.randn(n, h, generator=gen).bfloat16().to(gpu_device)
    weight = (torch.randn(v, h, generator=gen) * 0.2).bfloat16().to(gpu_device)
    labels = torch.randint(0, v, (n,), generator=gen).to(gpu_device)
    a = hidden.clone().requires_grad_(True)
    loss, _, _, _ = frozen_linear_ce_topk(a, weight, labels, top_k=3)
    loss.sum().backward()
    b = hidden.clone().requires_grad_(True)
    ref = tiled_linear_cross_entropy(b, weight, labels, reduction="sum", dtype=torch.bfloat16,
                                     weight_layout="vocab_first")
    ref.backward()
    torch.cuda.synchronize()
    torch.testing.assert_close(loss.sum(), ref, rtol=1e-4, atol=1e-2)
    denom = float(b.grad.float().abs().max())
    assert float((a.grad.float() - b.grad.float()).abs().max()) <= 1e-2 * denom


@pytest.mark.gpu
def test_ties_go_to_the_smaller_id(gpu_device):
    """All logits equal (zero hidden states): the top-k are ids 0 .. k-1, in
    every path of the scan (gather overflow on the first logits, rank merge
    with nothing to add afterwards)."""
    n, h, v, k = 5, 64, 40000, 7
    hidden = torch.zeros(n, h, dtype=torch.bfloat16, device=gpu_device)
    weight = torch.randn(v, h, generator=torch.Generator().manual_seed(1)).bfloat16().to(gpu_device)
    labels = torch.arange(n, device=gpu_device)
    loss, prob, vals, ids = frozen_linear_ce_topk(hidden, weight, labels, top_k=k)
    torch.cuda.synchronize()
    assert ids.tolist() == [list(range(k))] * n
    assert torch.count_nonzero(vals) == 0
    torch.testing.assert_close(loss.cpu(), torch.full((n,), float(torch.log(torch.tensor(float(v))))),
                               rtol=1e-5, atol=1e-5)


EXACT_CASES = [
    # name, rows, h, v, k, multiplier, panel_bytes (0 = default: one panel)
    ("k1_five_chunks", 70, 64, 70000, 1, 1.0, 0),
    ("k16_two_panels_two_chunks", 300, 64, 40000, 16, 1.0, 512 * 20480 * 4),
    ("k256_selection_rounds", 40, 64, 40000, 256, 0.5, 0),
    ("k16_many_panels", 130, 32, 20000, 16, 2.0, 256 * 2048 * 4),
    ("k256_many_panels", 257, 64, 33000, 256, 1.0, 512 * 4096 * 4),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", EXACT_CASES, ids=[c[0] for c in EXACT_CASES])
def test_selection_is_exact_on_exactly_representable_logits(gpu_device, case, set_panel_budget):
    """The selection isolated from matmul rounding: small-integer hidden states and
    weights in eighths make every product and every float32 partial sum exact, so
    the device's logits equal the oracle's bit for bit and the top-k ids and
    values must too, ties (there are thousands per row) going to the smaller id
    (at::topk semantics of the reference, fused_linear_ce_cuda.cu:1602 /
    dflash_linear_topk.py:100-158).  Covers rows spanning several 16384-logit
    chunks, several vocabulary panels, and k = 256 (selection rounds)."""
    name, n, h, v, k, mult, panel_bytes = case
    print("[case] exact top-k", name, flush=True)
    if panel_bytes:
        set_panel_budget(panel_bytes)
    gen = torch.Generator().manual_seed(len(name) * 7 + k)
    hidden = torch.randint(-3, 4, (n, h), generator=gen).to(torch.bfloat16)
    weight = (torch.randint(-8, 9, (v, h), generator=gen).float() / 8.0).to(torch.bfloat16)
    # a few rows with extreme ties: constant rows and rows with one distinct logit
    hidden[0] = 0
    if n > 2:
        hidden[1] = 0
        hidden[1, 0] = 1
    labels = torch.randint(0, v, (n,), generator=gen)
    loss, prob, vals, ids = frozen_linear_ce_topk(hidden.to(gpu_device), weight.to(gpu_device),
                                                  labels.to(gpu_device), top_k=k,
                                                  output_multiplier=mult)
    torch.cuda.synchronize()
    r_loss, _, r_vals, r_ids, _ = oracle.dense_ce_topk(hidden, weight, labels, k,
                                                       output_multiplier=mult)
    z = oracle._topk_logits(hidden, weight, mult, None, torch.float64)[0]
    assert bool((z == z.float().double()).all())          # the logits are float32-exact
    ties = int((z[:, :, None] == r_vals[:, None, -1:]).sum(dim=1).max())
    print("[case] logits tied with the k-th value in the worst row:", ties, flush=True)
    assert torch.equal(ids.cpu(), r_ids)
    assert torch.equal(vals.cpu().double(), r_vals)
    torch.testing.assert_close(loss.cpu().double(), r_loss, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("softcap,std", [(None, 0.2), (None, 2.5), (4.0, 0.5)])
def test_gradient_formed_in_the_forward_over_several_logits_panels(gpu_device, softcap, std,
                                                                   set_panel_budget):
    """bf16 operands the library takes: the forward also leaves d lse / d hidden (its
    grad_hidden contraction shows up in the forward's launch counts) and the backward is
    one pass over rows.  Four float32 logits panels, so most rows' maxima grow after their
    first panels were written and those are rescaled (std 2.5: by tens of nats).  Against
    the oracle and against the recomputing backward."""
    from turbo_dllm_amd import _lib, options
    print("[case] top-k gradient in the forward", softcap, std, flush=True)
    n, h, v, k = 520, 128, 4096, 8
    set_panel_budget(768 * 1024 * 4)
    gen = torch.Generator().manual_seed(17)
    hidden = torch.randn(n, h, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(v, h, generator=gen) * std).to(torch.bfloat16)
    labels = torch.randint(0, v, (n,), generator=gen)
    gl, gp, gv = (torch.randn(n, generator=gen), torch.randn(n, generator=gen),
                  torch.randn(n, k, generator=gen))
    grads = {}
    for mode in options.GRADIENT_MODES:
        x = hidden.to(gpu_device).requires_grad_(True)
        with options.gradient_mode(mode), _lib.kernel_profile() as prof:
            loss, prob, vals, ids = frozen_linear_ce_topk(
                x, weight.to(gpu_device), labels.to(gpu_device), top_k=k,
                output_multiplier=0.75, logit_softcap=softcap)
            torch.cuda.synchronize()
        assert prof.launches["grad_logits_panel"] == 4          # the float32 logits panels
        assert (prof.launches["grad_hidden_gemm"] > 0) == (mode == "forward")
        ((gl.to(gpu_device) * loss).sum() + (gp.to(gpu_device) * prob).sum()
         + (gv.to(gpu_device) * vals).sum()).backward()
        torch.cuda.synchronize()
        grads[mode] = (x.grad.cpu(), ids.cpu(), loss.detach().cpu())
    assert torch.equal(grads["forward"][1], grads["recompute"][1])
    assert torch.equal(grads["forward"][2], grads["recompute"][2])
    r_grad = oracle.dense_ce_topk_grad(hidden, weight, labels, grads["forward"][1], gl, gp, gv,
                                       output_multiplier=0.75, logit_softcap=softcap)
    for mode in options.GRADIENT_MODES:
        err = oracle.relative_max_error(grads[mode][0], r_grad)
        print("[case]", mode, "grad rel max err", f"{err:.2e}", flush=True)
        assert bool(torch.isfinite(grads[mode][0].float()).all())
        assert err <= 2e-2


@pytest.mark.gpu
def test_gradient_in_the_forward_backward_twice_and_no_gradient(gpu_device):
    """retain_graph: a second backward with other upstream gradients; and a forward whose
    hidden states need no gradient runs no gradient contraction."""
    from turbo_dllm_amd import _lib
    n, h, v, k = 300, 64, 2048, 4
    gen = torch.Generator().manual_seed(23)
    hidden = torch.randn(n, h, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(v, h, generator=gen) * 0.3).to(torch.bfloat16)
    labels = torch.randint(0, v, (n,), generator=gen)
    x = hidden.to(gpu_device).requires_grad_(True)
    loss, prob, vals, ids = frozen_linear_ce_topk(x, weight.to(gpu_device), labels.to(gpu_device),
                                                  top_k=k)
    for seed in (1, 2):
        g = torch.Generator().manual_seed(seed)
        gl, gp, gv = torch.randn(n, generator=g), torch.randn(n, generator=g), torch.randn(n, k, generator=g)
        x.grad = None
        ((gl.to(gpu_device) * loss).sum() + (gp.to(gpu_device) * prob).sum()
         + (gv.to(gpu_device) * vals).sum()).backward(retain_graph=True)
        r_grad = oracle.dense_ce_topk_grad(hidden, weight, labels, ids.cpu(), gl, gp, gv)
        assert oracle.relative_max_error(x.grad.cpu(), r_grad) <= 2e-2
    with _lib.kernel_profile() as prof:
        frozen_linear_ce_topk(hidden.to(gpu_device), weight.to(gpu_device),
                              labels.to(gpu_device), top_k=k)
        torch.cuda.synchronize()
    assert prof.launches["grad_hidden_gemm"] == 0
