"""Frozen-head forward KL: argument checks and the host path on the CPU (the
reference's own host cases), the device path against the float64 oracle."""

import pytest
import torch

import linear_ce_oracle as oracle
from turbo_dllm_amd.dflash_kl import frozen_linear_kl


def test_argument_checks():
    a, w = torch.randn(4, 8), torch.randn(11, 8)
    with pytest.raises(ValueError, match=r"\[tokens, hidden\]"):
        frozen_linear_kl(torch.randn(8), w, a, w)
    with pytest.raises(ValueError, match="token counts differ"):
        frozen_linear_kl(a, w, torch.randn(5, 8), w)
    with pytest.raises(ValueError, match=r"\[vocabulary, hidden\]"):
        frozen_linear_kl(a, torch.randn(8), a, w)
    with pytest.raises(ValueError, match="vocabularies differ"):
        frozen_linear_kl(a, w, a, torch.randn(12, 8))
    with pytest.raises(ValueError, match="draft head width"):
        frozen_linear_kl(a, torch.randn(11, 7), a, w)
    with pytest.raises(ValueError, match="teacher head width"):
        frozen_linear_kl(a, w, a, torch.randn(11, 7))
    with pytest.raises(ValueError, match="must be positive"):
        frozen_linear_kl(a, w, a, w, logit_softcap=0.0)


@pytest.mark.parametrize("seed,shapes,softcap", [(17, (7, 5, 6, 11), None),
                                                 (23, (5, 7, 9, 13), 2.5)])
def test_host_path_reference_cases(seed, shapes, softcap):
    """tests/unit/kernels/test_dflash_kl.py:13-76 of the reference."""
    n, hd, ht, v = shapes
    torch.manual_seed(seed)
    dh = torch.randn(n, hd, requires_grad=True)
    th, dw, tw = torch.randn(n, ht), torch.randn(v, hd), torch.randn(v, ht)
    scale = torch.randn(n)
    got = frozen_linear_kl(dh, dw, th, tw, logit_softcap=softcap)
    grad = torch.autograd.grad((got * scale).sum(), dh)[0]
    ref = oracle.dense_frozen_kl(dh.detach(), dw, th, tw, logit_softcap=softcap)
    ref_grad = oracle.dense_frozen_kl_grad(dh.detach(), dw, th, tw, scale, logit_softcap=softcap)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double(), ref, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(grad.double(), ref_grad, rtol=1e-4, atol=1e-6)


GPU_CASES = [
    # name, dtype, N, H_draft, H_teacher, V, softcap, weight std, loss tol, grad tol
    ("ref_bf16_seed31", torch.bfloat16, 7, 32, 48, 257, None, 1.0, 2e-2, 4e-2),
    ("ref_bf16_softcap_seed37", torch.bfloat16, 7, 32, 48, 257, 3.0, 1.0, 2e-2, 4e-2),
    ("f32_generic", torch.float32, 37, 33, 20, 301, None, 0.3, 2e-5, 2e-5),
    ("bf16_direct", torch.bfloat16, 300, 256, 128, 2304, None, 0.08, 2e-2, 2e-2),
    ("bf16_direct_softcap", torch.bfloat16, 129, 128, 192, 1536, 5.0, 0.2, 2e-2, 2e-2),
    ("bf16_mixed_engines", torch.bfloat16, 70, 128, 72, 1000, None, 0.15, 2e-2, 2e-2),
    ("f16_direct_two_panels", torch.float16, 520, 64, 64, 1024, None, 0.2, 2e-2, 2e-2),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", GPU_CASES, ids=[c[0] for c in GPU_CASES])
def test_device_path_matches_oracle(gpu_device, case, set_panel_budget):
    name, dtype, n, hd, ht, v, softcap, std, loss_tol, grad_tol = case
    print("[case]", name, flush=True)
    if "two_panels" in name:
        set_panel_budget(768 * 512 * 2)   # 512 columns per panel
    gen = torch.Generator().manual_seed({"ref_bf16_seed31": 31, "ref_bf16_softcap_seed37": 37}
                                        .get(name, len(name)))
    dh = torch.randn(n, hd, generator=gen).to(dtype)
    th = torch.randn(n, ht, generator=gen).to(dtype)
    dw = (torch.randn(v, hd, generator=gen) * std).to(dtype)
    tw = (torch.randn(v, ht, generator=gen) * std).to(dtype)
    scale = torch.randn(n, generator=gen)
    x = dh.to(gpu_device).requires_grad_(True)
    got = frozen_linear_kl(x, dw.to(gpu_device), th.to(gpu_device), tw.to(gpu_device),
                           logit_softcap=softcap)
    (got * scale.to(gpu_device)).sum().backward()
    torch.cuda.synchronize()
    ref = oracle.dense_frozen_kl(dh, dw, th, tw, logit_softcap=softcap)
    ref_grad = oracle.dense_frozen_kl_grad(dh, dw, th, tw, scale, logit_softcap=softcap)
    assert got.dtype == torch.float32 and got.shape == (n,)
    assert x.grad.dtype == dtype and x.grad.shape == (n, hd)
    print("[case] loss max abs err", float((got.cpu().double() - ref).abs().max()),
          "ref max", float(ref.max()), "grad rel max err",
          oracle.relative_max_error(x.grad.cpu(), ref_grad), flush=True)
    torch.testing.assert_close(got.cpu().double(), ref, rtol=loss_tol, atol=loss_tol)
    assert oracle.relative_max_error(x.grad.cpu(), ref_grad) <= grad_tol


@pytest.mark.gpu
def test_same_head_gives_zero(gpu_device):
    gen = torch.Generator().manual_seed(9)
    h = torch.randn(200, 128, generator=gen).bfloat16().to(gpu_device)
    w = (torch.randn(1536, 128, generator=gen) * 0.2).bfloat16().to(gpu_device)
    x = h.clone().requires_grad_(True)
    got = frozen_linear_kl(x, w, h, w)
    got.sum().backward()
    torch.cuda.synchronize()
    assert float(got.abs().max()) < 2e-3
    assert float(x.grad.float().abs().max()) < 2e-2 * float(w.float().abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,hd,ht,v,softcap", [
    (torch.bfloat16, 128, 192, 4096, None),     # direct engine, panels staged through LDS
    (torch.bfloat16, 128, 128, 2048, 6.0),
    (torch.float16, 72, 72, 1000, None),        # staged engine, plain loads of the panel
    (torch.float32, 33, 40, 301, None),
])
def test_kept_teacher_probabilities_give_the_same_gradient(gpu_device, dtype, hd, ht, v, softcap,
                                                           set_panel_budget):
    """Where the gradient cannot be formed in the forward (soft cap, f16, float32) the
    default keeps the teacher probabilities of the whole vocabulary from the forward to
    the backward (5 contractions per step); gradient mode "recompute" produces them a
    second time (6).  Same producer, same values: the gradients agree bit for bit, over
    several vocabulary panels.  Which one ran is read from the launch counts of the
    backward, run on this thread through the shim.  (The first case is one the forward
    that leaves the gradient takes: there the default agrees within rounding, and the
    shim-level comparison still holds.)"""
    from turbo_dllm_amd import _lib, options
    from turbo_dllm_amd import chunked_linear_ce_native as native
    print("[case] kept teacher probabilities", dtype, hd, ht, v, softcap, flush=True)
    m = 300
    set_panel_budget(512 * 512 * 2)          # panels of 512 columns
    gen = torch.Generator().manual_seed(v)
    ops = [torch.randn(m, hd, generator=gen), torch.randn(v, hd, generator=gen) * 0.2,
           torch.randn(m, ht, generator=gen), torch.randn(v, ht, generator=gen) * 0.2]
    ops = [t.to(dtype).to(gpu_device) for t in ops]
    go = torch.rand(m, generator=gen).to(gpu_device)
    grads = {}
    for mode in options.GRADIENT_MODES:
        x = ops[0].clone().requires_grad_(True)
        with options.gradient_mode(mode):
            losses = frozen_linear_kl(x, ops[1], ops[2], ops[3], logit_softcap=softcap)
        losses.backward(go)
        torch.cuda.synchronize()
        grads[mode] = (losses.detach().cpu(), x.grad.cpu())
    if native.kl_gradient_in_forward_supported(ops[0], ops[1], ops[2], float(softcap or 0.0)):
        # (the two paths round different things to bf16: teacher probabilities there,
        # exp2(z2 - tile maximum) of both heads here; each is within a few 1e-3 of the loss)
        torch.testing.assert_close(grads["forward"][0], grads["recompute"][0], rtol=1e-2, atol=5e-2)
        assert oracle.relative_max_error(grads["forward"][1], grads["recompute"][1].float()) <= 1e-2
    else:
        assert torch.equal(grads["forward"][0], grads["recompute"][0])
        assert torch.equal(grads["forward"][1], grads["recompute"][1])
    # through the shim on this thread: the backward that reads the kept panel launches the
    # panel kernels once per panel (the draft pass), the other twice (teacher, then draft)
    cap = float(softcap or 0.0)
    losses, dlse, tlse, kept = native.dflash_kl_forward(*ops, cap, keep_teacher_probabilities=True)
    assert kept.dtype == torch.uint8 and kept.numel() == native.kl_teacher_probabilities_bytes(
        ops[0], ops[1], ops[2])
    counts = {}
    for name, panel in (("kept", kept), ("again", None)):
        with _lib.kernel_profile() as prof:
            g = native.dflash_kl_backward(*ops, dlse, tlse, go, cap, teacher_probabilities=panel)
            torch.cuda.synchronize()
        counts[name] = prof.launches["grad_logits_panel"]
        assert torch.equal(g.cpu(), grads["recompute"][1])
    assert counts["again"] == 2 * counts["kept"] and counts["kept"] >= 1
    if dtype == torch.bfloat16:
        assert counts["kept"] == v // 512          # several vocabulary panels
    with pytest.raises(RuntimeError, match="teacher_probabilities"):
        native.dflash_kl_backward(*ops, dlse, tlse, go, cap, teacher_probabilities=kept[:16])


@pytest.mark.gpu
@pytest.mark.parametrize("m,hd,ht,v,std,softcap", [
    (300, 128, 192, 4096, 0.2, None),
    (700, 64, 64, 2048, 1.5, None),  # logits tens of nats apart: entries far below their tile maximum
    (1, 256, 128, 576, 0.3, None),
    (300, 128, 128, 2048, 0.3, 12.0),
    (520, 64, 128, 4096, 3.0, 30.0),  # logits deep in the cap on both sides
])
def test_gradient_formed_in_the_forward(gpu_device, m, hd, ht, v, std, softcap,
                                        set_panel_budget):
    """bf16 (with a soft cap between 10 and 40, or none): the draft pass of the forward leaves
    exp2(z2 - tile maximum), and d loss / d draft_hidden is contracted in the forward (its grad_hidden
    contraction shows in the forward's launch counts); the backward scales rows.  Loss and
    gradient against the float64 oracle; the loss is held to the plain forward's distance
    from the oracle (the two round different things to bf16 on their way through memory:
    teacher probabilities there, exp2(z2 - tile maximum) of both heads here)."""
    from turbo_dllm_amd import _lib, options
    print("[case] KL gradient in the forward", m, hd, ht, v, std, softcap, flush=True)
    set_panel_budget(512 * 512 * 2)
    gen = torch.Generator().manual_seed(m + v)
    cpu = [torch.randn(m, hd, generator=gen), torch.randn(v, hd, generator=gen) * std,
           torch.randn(m, ht, generator=gen), torch.randn(v, ht, generator=gen) * std]
    cpu = [t.to(torch.bfloat16) for t in cpu]
    ops = [t.to(gpu_device) for t in cpu]
    go = torch.rand(m, generator=gen) + 0.1
    x = ops[0].clone().requires_grad_(True)
    with _lib.kernel_profile() as prof:
        losses = frozen_linear_kl(x, ops[1], ops[2], ops[3], logit_softcap=softcap)
        torch.cuda.synchronize()
    assert prof.launches["grad_hidden_gemm"] == 1
    losses.backward(go.to(gpu_device))
    torch.cuda.synchronize()
    ref_loss = oracle.dense_frozen_kl(cpu[0], cpu[1], cpu[2], cpu[3], logit_softcap=softcap)
    with options.gradient_mode("recompute"):
        plain = frozen_linear_kl(ops[0], ops[1], ops[2], ops[3], logit_softcap=softcap)
    err_here = float((losses.detach().cpu().double() - ref_loss).abs().max())
    err_plain = float((plain.cpu().double() - ref_loss).abs().max())
    print("[case] loss max abs err", f"{err_here:.2e}", "plain forward", f"{err_plain:.2e}",
          flush=True)
    assert err_here <= max(2.0 * err_plain, 2e-3)
    torch.testing.assert_close(losses.detach().cpu().double(), ref_loss, rtol=2e-2, atol=1e-3)
    ref_grad = oracle.dense_frozen_kl_grad(cpu[0], cpu[1], cpu[2], cpu[3], go,
                                           logit_softcap=softcap)
    err = oracle.relative_max_error(x.grad.cpu(), ref_grad)
    print("[case] grad rel max err", f"{err:.2e}", flush=True)
    assert bool(torch.isfinite(x.grad.float()).all())
    assert err <= 2e-2
