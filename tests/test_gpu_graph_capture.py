"""The entry points can be recorded into a HIP graph: they launch only kernels
and device-to-device copies on the stream they are given (zero fills are
kernels, not memsets), allocate nothing themselves and never synchronise.

The graph is replayed several times with new input contents, eager work and
synchronisations in between, and every replay is compared with the eager
result of the same inputs, bit for bit.
"""

import pytest
import torch

from turbo_dllm_amd import chunked_linear_ce_native as native

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,h,v", [(300, 128, 1536), (129, 72, 1025)])
def test_forward_backward_graph_replays_match_eager(gpu_device, n, h, v):
    print("[case] graph capture", n, h, v, flush=True)
    dev = gpu_device
    gen = torch.Generator().manual_seed(n)

    def make():
        hidden = torch.randn(n, h, generator=gen).bfloat16()
        labels = torch.randint(0, v, (n,), generator=gen)
        labels[torch.rand(n, generator=gen) < 0.2] = -100
        return hidden, labels

    weight = (torch.randn(v, h, generator=gen) * 0.2).bfloat16().to(dev)
    kw = dict(row_block_size=0, ignore_index=-100, exclude_index=-1, logit_softcap=0.0,
              compute_dtype=torch.bfloat16, weight_dim_first=False)
    go = torch.ones(1, device=dev)

    def run(hidden, labels):
        losses, lse, count = native.forward(hidden, weight, None, labels, **kw)
        dh, dw, _ = native.backward(hidden, weight, None, labels, lse, count, go,
                                    reduction="mean", **kw)
        return losses, dh, dw

    static_hidden = torch.zeros(n, h, dtype=torch.bfloat16, device=dev)
    static_labels = torch.zeros(n, dtype=torch.long, device=dev)
    first = make()
    static_hidden.copy_(first[0])
    static_labels.copy_(first[1])
    run(static_hidden, static_labels)            # warm-up: one-time kernel attributes
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = run(static_hidden, static_labels)
    torch.cuda.synchronize()

    for replay in range(4):
        hidden, labels = first if replay == 0 else make()
        static_hidden.copy_(hidden)
        static_labels.copy_(labels)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs]
        eager = run(hidden.to(dev), labels.to(dev))      # eager work between replays
        torch.cuda.synchronize()
        for name, a, b in zip(("losses", "grad_hidden", "grad_weight"), got, eager):
            assert torch.equal(a, b), (replay, name)


@pytest.mark.parametrize("n,h,v", [(700, 128, 1536), (260, 72, 1025)])
def test_whole_loss_with_device_row_count_replays_for_any_mask(gpu_device, n, h, v):
    """Compaction, fused gather, forward and backward of the masked-token loss in
    ONE graph: the count of loss-bearing rows never leaves the device, so the
    same graph serves masks with different counts (down to none at all).  Every
    replay is compared bit for bit with an eager run of the same calls and, for
    the weighted sum, with the synchronising path."""
    print("[case] whole-loss graph capture", n, h, v, flush=True)
    dev = gpu_device
    gen = torch.Generator().manual_seed(n + 1)
    weight = (torch.randn(v, h, generator=gen) * 0.2).bfloat16().to(dev)
    go = torch.full((1,), 0.5, device=dev)
    kw = dict(ignore_index=-100, exclude_index=3, logit_softcap=0.0, logit_multiplier=0.5)

    def make(rate):
        hidden = torch.randn(n, h, generator=gen).bfloat16()
        labels = torch.randint(4, v, (n,), generator=gen)
        labels[torch.rand(n, generator=gen) < rate] = -100
        weights = torch.rand(n, generator=gen) + 0.5
        return hidden, labels, weights

    def run(hidden, labels, weights):
        row_idx, count = native.compact_rows_device(labels, -100)
        rows, targets, w = native.gather_loss_rows(hidden, labels, weights, row_idx, count, -100)
        _, lse, _, total = native.masked_loss_forward(
            rows, weight, None, targets, w, m=n, row_idx=row_idx, row_count=count, n_out=n,
            want_losses=False, want_sum=True, **kw)
        dh, dw, _ = native.masked_loss_backward(
            rows, weight, None, targets, w, lse, None, go, reduction="sum", m=n,
            row_idx=row_idx, row_count=count, n_out=n, **kw)
        return total, dh, dw, count

    static = [torch.zeros(n, h, dtype=torch.bfloat16, device=dev),
              torch.zeros(n, dtype=torch.long, device=dev),
              torch.zeros(n, dtype=torch.float32, device=dev)]
    first = make(0.5)
    for s, t in zip(static, first):
        s.copy_(t)
    run(*static)                                  # warm-up: one-time kernel attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = run(*static)
    torch.cuda.synchronize()

    for replay, rate in enumerate((0.5, 0.05, 0.97, 1.0, 0.0)):
        case = first if replay == 0 else make(rate)
        for s, t in zip(static, case):
            s.copy_(t)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs]
        eager = run(*[t.to(dev) for t in case])   # eager work between replays
        torch.cuda.synchronize()
        assert int(got[3]) == int((case[1] != -100).sum()), replay
        for name, a, b in zip(("weighted_sum", "grad_hidden", "grad_weight", "count"), got, eager):
            assert torch.equal(a, b), (replay, rate, name)
        # the synchronising path (exact launch sizes) computes the same sum
        hidden, labels, weights = (t.to(dev) for t in case)
        idx, m = native.compact_rows(labels, -100)
        _, _, _, total = native.masked_loss_forward(
            native.gather_rows(hidden, idx), weight, None, native.gather_rows(labels, idx),
            native.gather_rows(weights, idx), row_idx=idx if m < n else None, n_out=n,
            want_losses=False, want_sum=True, **kw)
        assert torch.equal(total, got[0]), (replay, rate)


@pytest.mark.parametrize("n,hd,ht,v,softcap", [(300, 128, 64, 1536, 0.0), (130, 72, 96, 1025, 5.0)])
def test_frozen_kl_graph_replays_match_eager(gpu_device, n, hd, ht, v, softcap, set_panel_budget):
    """The KL of two frozen heads, forward and backward, from one graph: its
    loss is accumulated per vocabulary tile and merged in a fixed order (no
    float atomics), so replays and eager runs agree bit for bit, and so do
    repeated eager runs."""
    print("[case] KL graph capture", n, hd, ht, v, softcap, flush=True)
    dev = gpu_device
    set_panel_budget(512 * 512 * 2)      # several vocabulary panels
    gen = torch.Generator().manual_seed(n + v)
    draft_w = (torch.randn(v, hd, generator=gen) * 0.2).bfloat16().to(dev)
    teacher_w = (torch.randn(v, ht, generator=gen) * 0.2).bfloat16().to(dev)

    def make():
        return (torch.randn(n, hd, generator=gen).bfloat16(),
                torch.randn(n, ht, generator=gen).bfloat16(),
                torch.rand(n, generator=gen) + 0.5)

    def run(draft_h, teacher_h, go):
        losses, draft_lse, teacher_lse = native.dflash_kl_forward(draft_h, draft_w, teacher_h,
                                                                  teacher_w, softcap)
        grad = native.dflash_kl_backward(draft_h, draft_w, teacher_h, teacher_w, draft_lse,
                                         teacher_lse, go, softcap)
        return losses, grad

    static = [torch.zeros(n, hd, dtype=torch.bfloat16, device=dev),
              torch.zeros(n, ht, dtype=torch.bfloat16, device=dev),
              torch.zeros(n, dtype=torch.float32, device=dev)]
    first = make()
    for s, t in zip(static, first):
        s.copy_(t)
    run(*static)                                  # warm-up: one-time kernel attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = run(*static)
    torch.cuda.synchronize()
    for replay in range(4):
        case = first if replay == 0 else make()
        for s, t in zip(static, case):
            s.copy_(t)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs]
        eager = run(*[t.to(dev) for t in case])   # eager work between replays
        again = run(*[t.to(dev) for t in case])
        torch.cuda.synchronize()
        for name, a, b, c in zip(("losses", "grad_hidden"), got, eager, again):
            assert torch.equal(a, b), (replay, name)
            assert torch.equal(b, c), (replay, name, "eager runs differ")


@pytest.mark.parametrize("n,h,v", [(700, 128, 1536)])
def test_gradients_formed_in_the_forward_graph_replays_match_eager(gpu_device, n, h, v,
                                                                   set_panel_budget):
    """The forward that leaves the gradients, and the scaling by the upstream
    gradient, from one graph: the decision to redo a block of rows with exact row
    maxima is taken on the device (the second try's launches are recorded and do
    nothing unless asked), so one graph serves inputs that need it and inputs that
    do not."""
    print("[case] fused-gradient graph capture", n, h, v, flush=True)
    dev = gpu_device
    set_panel_budget(256 * v * 2)          # one token tile per block: three blocks
    gen = torch.Generator().manual_seed(n)
    weight = (torch.randn(v, h, generator=gen) * 0.2).bfloat16().to(dev)

    def make(far_rows):
        hidden = torch.randn(n, h, generator=gen).bfloat16()
        labels = torch.randint(0, v, (n,), generator=gen)
        labels[torch.rand(n, generator=gen) < 0.2] = -100
        for r in range(0, n, 5) if far_rows else ():
            # a logit ~120 on another column than the label's: outside the window
            w = weight[(int(labels[r]) + 1) % v].float().cpu()
            hidden[r] = (w * (120.0 / float(w @ w))).bfloat16()
        return hidden, labels

    go = torch.full((1,), 0.75, device=dev)

    def run(hidden, labels):
        losses, lse, count, dh32, dw32 = native.forward_with_gradients(
            hidden, weight, labels, ignore_index=-100, exclude_index=-1, logit_softcap=0.0,
            compute_weight_grad=True)
        dh, dw = native.apply_grad_output(dh32, dw32, go, count, reduction="mean",
                                          dtype=torch.bfloat16)
        return losses, dh, dw

    static_hidden = torch.zeros(n, h, dtype=torch.bfloat16, device=dev)
    static_labels = torch.zeros(n, dtype=torch.long, device=dev)
    first = make(False)
    static_hidden.copy_(first[0])
    static_labels.copy_(first[1])
    run(static_hidden, static_labels)            # warm-up: one-time kernel attributes
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = run(static_hidden, static_labels)
    torch.cuda.synchronize()

    for replay in range(5):
        hidden, labels = first if replay == 0 else make(far_rows=replay in (2, 3))
        static_hidden.copy_(hidden)
        static_labels.copy_(labels)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs]
        eager = run(hidden.to(dev), labels.to(dev))      # eager work between replays
        torch.cuda.synchronize()
        for name, a, b in zip(("losses", "grad_hidden", "grad_weight"), got, eager):
            assert torch.equal(a, b), (replay, name)
        assert torch.isfinite(got[0]).all() and torch.isfinite(got[1].float()).all()


def _replay_against_eager(dev, run, make, static, names, replays=4):
    """Captures run(*static) once, then replays it for fresh inputs with eager work and
    synchronisations in between; every replay must equal the eager result bit for bit."""
    first = make()
    for s, t in zip(static, first):
        s.copy_(t)
    run(*static)                                  # warm-up: one-time kernel attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = run(*static)
    torch.cuda.synchronize()
    for replay in range(replays):
        case = first if replay == 0 else make()
        for s, t in zip(static, case):
            s.copy_(t)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs]
        eager = run(*[t.to(dev) for t in case])   # eager work between replays
        torch.cuda.synchronize()
        for name, a, b in zip(names, got, eager):
            assert torch.equal(a, b), (replay, name)


def test_frozen_kl_gradient_in_the_forward_graph_replays_match_eager(gpu_device, set_panel_budget):
    """The KL forward that leaves d loss / d hidden, and the row scaling that is its
    backward, from one graph (kernels and device-to-device work only)."""
    print("[case] KL gradient-in-forward graph capture", flush=True)
    dev = gpu_device
    n, hd, ht, v = 300, 128, 64, 1536
    set_panel_budget(512 * 512 * 2)
    gen = torch.Generator().manual_seed(5)
    draft_w = (torch.randn(v, hd, generator=gen) * 0.2).bfloat16().to(dev)
    teacher_w = (torch.randn(v, ht, generator=gen) * 0.2).bfloat16().to(dev)

    def make():
        return (torch.randn(n, hd, generator=gen).bfloat16(),
                torch.randn(n, ht, generator=gen).bfloat16(),
                torch.rand(n, generator=gen) + 0.5)

    def run(draft_h, teacher_h, go):
        losses, _, _, unit = native.dflash_kl_forward_with_gradient(draft_h, draft_w, teacher_h,
                                                                    teacher_w, 0.0)
        grad, _ = native.apply_grad_output(unit, None, go, None, reduction="none",
                                           dtype=torch.bfloat16)
        return losses, grad

    static = [torch.zeros(n, hd, dtype=torch.bfloat16, device=dev),
              torch.zeros(n, ht, dtype=torch.bfloat16, device=dev),
              torch.zeros(n, dtype=torch.float32, device=dev)]
    _replay_against_eager(dev, run, make, static, ("losses", "grad_hidden"))


def test_ce_topk_gradient_in_the_forward_graph_replays_match_eager(gpu_device, set_panel_budget):
    """Frozen-head cross entropy with top-k, d lse / d hidden formed in the forward over
    several float32 logits panels (with the rescaling of panels written before a row's
    maximum grew), and the row pass that is its backward, from one graph."""
    print("[case] CE top-k gradient-in-forward graph capture", flush=True)
    dev = gpu_device
    n, h, v, k = 260, 128, 4096, 8
    set_panel_budget(512 * 1024 * 4)
    gen = torch.Generator().manual_seed(6)
    weight = (torch.randn(v, h, generator=gen) * 0.5).bfloat16().to(dev)

    def make():
        return (torch.randn(n, h, generator=gen).bfloat16(),
                torch.randint(0, v, (n,), generator=gen),
                torch.randn(n, generator=gen), torch.randn(n, generator=gen),
                torch.randn(n, k, generator=gen))

    def run(hidden, labels, gl, gp, gv):
        loss, prob, vals, ids, _, unit = native.dflash_ce_topk_forward_with_gradient(
            hidden, weight, labels, top_k=k, output_multiplier=0.8, logit_softcap=0.0)
        grad = native.dflash_ce_topk_apply_gradient(unit, hidden, weight, labels, prob, ids, gl, gp,
                                                    gv, output_multiplier=0.8, logit_softcap=0.0)
        return loss, vals, ids, grad

    static = [torch.zeros(n, h, dtype=torch.bfloat16, device=dev),
              torch.zeros(n, dtype=torch.long, device=dev),
              torch.zeros(n, device=dev), torch.zeros(n, device=dev), torch.zeros(n, k, device=dev)]
    _replay_against_eager(dev, run, make, static, ("loss", "top_values", "top_ids", "grad_hidden"))
