"""Streaming soft embedding: argument checks and the host path on the CPU, the
device path against dense float64 softmax(h W^T) W on the GPU."""

import pytest
import torch

import linear_ce_oracle as oracle

from turbo_dllm_amd.streaming_soft_embedding import (
    streaming_soft_embedding,
    streaming_soft_embedding_from_shards,
)


def dense(hidden, weight, softcap=None, scale=1.0):
    return oracle.dense_soft_embedding(hidden, weight, logit_softcap=softcap, embedding_scale=scale)


def rel_max(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max())


def test_argument_checks():
    h = torch.randn(3, 8)
    w = torch.randn(11, 8)
    kw = dict(row_chunk_size=2, vocab_chunk_size=4)
    with pytest.raises(ValueError, match="at least two dimensions"):
        streaming_soft_embedding(torch.randn(8), w, **kw)
    with pytest.raises(ValueError, match="chunk sizes must be positive"):
        streaming_soft_embedding(h, w, row_chunk_size=0, vocab_chunk_size=4)
    with pytest.raises(ValueError, match="at least one vocabulary weight shard"):
        streaming_soft_embedding_from_shards(h, (), **kw)
    with pytest.raises(ValueError, match="two-dimensional"):
        streaming_soft_embedding(h, torch.randn(8), **kw)
    with pytest.raises(ValueError, match="does not match hidden"):
        streaming_soft_embedding(h, torch.randn(11, 7), **kw)
    with pytest.raises(ValueError, match="logit_softcap must be positive"):
        streaming_soft_embedding(h, w, logit_softcap=0.0, **kw)
    with pytest.raises(RuntimeError, match="tensor-parallel"):
        streaming_soft_embedding(h, w, tensor_parallel_size=2, **kw)


@pytest.mark.parametrize("softcap,scale", [(None, 1.0), (2.0, 3.0)])
def test_host_path_matches_dense(softcap, scale):
    torch.manual_seed(0)
    h = torch.randn(2, 5, 8)
    w = torch.randn(13, 8)
    got = streaming_soft_embedding(h, w, row_chunk_size=3, vocab_chunk_size=4,
                                   logit_softcap=softcap, embedding_scale=scale)
    assert got.shape == h.shape and got.dtype == h.dtype and not got.requires_grad
    assert rel_max(got, dense(h, w, softcap, scale)) < 1e-5
    shards = streaming_soft_embedding_from_shards(h, (w[:6], w[6:]), row_chunk_size=4,
                                                  vocab_chunk_size=5, logit_softcap=softcap,
                                                  embedding_scale=scale)
    assert rel_max(shards, got) < 1e-6
    empty = streaming_soft_embedding(torch.zeros(0, 8), w, row_chunk_size=3, vocab_chunk_size=4)
    assert empty.shape == (0, 8)


GPU_CASES = [
    ("f32_generic", torch.float32, (37, 33), 301, None, 1.0, 2e-5),
    ("bf16_staged_h72", torch.bfloat16, (61, 72), 1025, None, 1.0, 2e-2),
    ("bf16_direct", torch.bfloat16, (3, 100, 256), 2304, None, 1.0, 2e-2),
    ("bf16_direct_softcap_scale", torch.bfloat16, (129, 128), 1536, 5.0, 16.0, 2e-2),
    ("f16_direct", torch.float16, (70, 64), 1000, None, 0.5, 2e-2),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", GPU_CASES, ids=[c[0] for c in GPU_CASES])
def test_device_path_matches_dense(gpu_device, case):
    name, dtype, shape, v, softcap, scale, tol = case
    print("[case]", name, flush=True)
    gen = torch.Generator().manual_seed(len(name))
    h = torch.randn(*shape, generator=gen).to(dtype)
    w = (torch.randn(v, shape[-1], generator=gen) * (3.0 / shape[-1] ** 0.5)).to(dtype)
    got = streaming_soft_embedding(h.to(gpu_device), w.to(gpu_device), row_chunk_size=64,
                                   vocab_chunk_size=256, logit_softcap=softcap,
                                   embedding_scale=scale)
    torch.cuda.synchronize()
    assert got.shape == h.shape and got.dtype == dtype
    err = rel_max(got.cpu(), dense(h, w, softcap, scale))
    print("[case] rel max err", f"{err:.2e}", flush=True)
    assert err <= tol
    two = streaming_soft_embedding_from_shards(
        h.to(gpu_device), (w[: v // 2].to(gpu_device), w[v // 2:].to(gpu_device)),
        row_chunk_size=64, vocab_chunk_size=256, logit_softcap=softcap, embedding_scale=scale)
    assert torch.equal(two, got)


@pytest.mark.gpu
@pytest.mark.parametrize("softcap,tiles_per_block,std", [
    (30.0, 0, 3.0),      # the production cap, one block of rows
    (30.0, 1, 3.0),      # three blocks of rows
    (30.0, 0, 60.0),     # logits far into the cap on both sides: exp(z - cap) spans exp(-60)..1
    (40.0, 2, 8.0),      # the largest cap that sequence takes
    (50.0, 0, 8.0),      # beyond it, and without a cap: one emitting pass (entries relative
    (None, 1, 3.0),      # to exact tile maxima), an elementwise normalisation, the contraction
    (None, 0, 40.0),     # logits hundreds of nats apart
])
def test_soft_embedding_takes_two_contractions(gpu_device, softcap, tiles_per_block, std):
    """Capped logits lie in [-cap, cap]: exp(z - cap) needs no row maximum, so the
    device path writes it to the panel in one contraction and normalises after the
    second.  Without a usable cap one pass over the head emits exp2(z2 - tile maximum)
    with the softmax partials, and the entries are normalised per (token, tile) before
    the second contraction.  No statistics pass either way (which sequence ran is read
    from the library's per-class launch counts)."""
    from turbo_dllm_amd import _lib, options
    print("[case] capped soft embedding", softcap, tiles_per_block, std, flush=True)
    m, hdim, v = 700, 128, 2048
    gen = torch.Generator().manual_seed(int(softcap or 0) + tiles_per_block)
    h = torch.randn(m, hdim, generator=gen).to(torch.bfloat16)
    w = (torch.randn(v, hdim, generator=gen) * (std / hdim ** 0.5)).to(torch.bfloat16)
    with options.panel_budget(tiles_per_block * 256 * v * 2), _lib.kernel_profile() as prof:
        got = streaming_soft_embedding(h.to(gpu_device), w.to(gpu_device), row_chunk_size=64,
                                       vocab_chunk_size=256, logit_softcap=softcap,
                                       embedding_scale=2.0)
        torch.cuda.synchronize()
    blocks = 1 if tiles_per_block == 0 else -(-m // (256 * tiles_per_block))
    capped = softcap is not None and softcap <= 40.0
    assert prof.launches["forward_stats"] == 0
    assert prof.launches["exp_logits_panel"] == (blocks if capped else 0)
    assert prof.launches["grad_logits_panel"] == (0 if capped else blocks)   # the emitting pass
    assert prof.launches["grad_hidden_gemm"] == blocks
    assert bool(torch.isfinite(got.float()).all())
    err = rel_max(got.cpu(), dense(h, w, softcap, 2.0))
    print("[case] rel max err", f"{err:.2e}", flush=True)
    assert err <= 2e-2
