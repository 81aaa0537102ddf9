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
