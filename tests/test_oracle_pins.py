"""Pins the CPU oracle before anything is compared against it.

Each oracle function is checked against something it does not itself call: a
library routine (F.cross_entropy, autograd, torch.nonzero), a brute-force
Python loop, a closed form, or the committed fixtures.  The cases are chosen so
that a plausible slip (dropped bias, soft cap after the exclusion, onehot with
the wrong sign, scale missing from mean, transposed grad_weight, ignored rows
counted in the mean) fails at least one test.
"""

import math
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import linear_ce_oracle as oracle

GOLDEN = Path(__file__).resolve().parent / "golden" / "linear_ce_cases.npz"


def _golden_cases():
    data = np.load(GOLDEN, allow_pickle=False)
    for entry in data["__cases__"]:
        name, softcap, exclude = str(entry).split("|")
        softcap = float(softcap.split("=")[1])
        exclude = int(exclude.split("=")[1])

        def get(key, _name=name):
            full = f"{_name}/{key}"
            return torch.from_numpy(data[full]) if full in data.files else None

        yield name, (softcap or None), (exclude if exclude >= 0 else None), get


@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_oracle_matches_golden_fixtures(reduction):
    seen = 0
    for name, softcap, exclude, get in _golden_cases():
        hidden, weight, labels, bias = get("hidden"), get("weight"), get("labels"), get("bias")
        loss = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, reduction=reduction,
                                      exclude_index=exclude, logit_softcap=softcap)
        torch.testing.assert_close(loss, get(f"loss_{reduction}"), atol=1e-11, rtol=1e-11,
                                   msg=f"{name} loss")
        go = get("grad_out") if reduction == "none" else None
        dh, dw, db = oracle.dense_linear_ce_grads(
            hidden, weight, labels, go, bias=bias, reduction=reduction, exclude_index=exclude,
            logit_softcap=softcap)
        torch.testing.assert_close(dh, get(f"dh_{reduction}"), atol=1e-11, rtol=1e-10)
        torch.testing.assert_close(dw, get(f"dw_{reduction}"), atol=1e-11, rtol=1e-10)
        if bias is not None:
            torch.testing.assert_close(db, get(f"db_{reduction}"), atol=1e-11, rtol=1e-10)
        seen += 1
    assert seen == 6


def test_oracle_matches_library_cross_entropy_and_autograd_bf16_inputs():
    # the shape of the reference's bf16 device test (test_tiled_linear_cross_entropy.py:303-354)
    torch.manual_seed(52)
    hidden = (torch.randn(31, 96) * 0.1).bfloat16()
    weight = (torch.randn(1025, 96) * 0.1).bfloat16()
    bias = (torch.randn(1025) * 0.1).bfloat16()
    labels = torch.randint(0, 1024, (31,))
    labels[::5] = -100
    h = hidden.double().requires_grad_(True)
    w = weight.double().requires_grad_(True)
    b = bias.double().requires_grad_(True)
    logits = h @ w.t() + b
    logits = logits + torch.zeros(1025, dtype=torch.float64).index_fill_(
        0, torch.tensor([1024]), -float("inf"))
    ref = F.cross_entropy(logits, labels, reduction="mean", ignore_index=-100)
    ref.backward()
    got = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, exclude_index=1024)
    torch.testing.assert_close(got, ref.detach(), atol=1e-12, rtol=1e-12)
    dh, dw, db = oracle.dense_linear_ce_grads(hidden, weight, labels, bias=bias,
                                              exclude_index=1024)
    torch.testing.assert_close(dh, h.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(dw, w.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(db, b.grad, atol=1e-12, rtol=1e-10)
    assert torch.count_nonzero(dw[1024]) == 0


def test_oracle_brute_force_tiny():
    torch.manual_seed(3)
    n, h, v, cap, excl = 4, 3, 6, 1.5, 2
    hidden = torch.randn(n, h, dtype=torch.float64)
    weight = torch.randn(v, h, dtype=torch.float64)
    bias = torch.randn(v, dtype=torch.float64)
    labels = torch.tensor([0, -100, 5, 3])
    expect = []
    for r in range(n):
        if labels[r] == -100:
            expect.append(0.0)
            continue
        zs = []
        for c in range(v):
            z = sum(float(hidden[r, k]) * float(weight[c, k]) for k in range(h)) + float(bias[c])
            zs.append(cap * math.tanh(z / cap))
        denom = sum(math.exp(z) for c, z in enumerate(zs) if c != excl)
        expect.append(math.log(denom) - zs[int(labels[r])])
    got = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, reduction="none",
                                 exclude_index=excl, logit_softcap=cap)
    torch.testing.assert_close(got, torch.tensor(expect, dtype=torch.float64), atol=1e-12,
                               rtol=1e-12)
    mean = oracle.dense_linear_ce(hidden, weight, labels, bias=bias, reduction="mean",
                                  exclude_index=excl, logit_softcap=cap)
    assert abs(float(mean) - sum(expect) / 3) < 1e-12  # ignored row not in the denominator


def test_oracle_closed_forms():
    # zero weights -> uniform softmax: loss = log V, and log(V-1) with one column excluded
    hidden = torch.randn(5, 8, dtype=torch.float64)
    weight = torch.zeros(17, 8, dtype=torch.float64)
    labels = torch.tensor([0, 3, 16, 7, 9])
    loss = oracle.dense_linear_ce(hidden, weight, labels, reduction="none")
    torch.testing.assert_close(loss, torch.full((5,), math.log(17), dtype=torch.float64))
    loss = oracle.dense_linear_ce(hidden, weight, labels.clamp(max=15), reduction="none",
                                  exclude_index=16)
    torch.testing.assert_close(loss, torch.full((5,), math.log(16), dtype=torch.float64))
    # without soft cap every row of the logit gradient sums to zero -> grad_bias sums to 0
    # and grad_hidden of a row equals sum_v g_v W_v
    torch.manual_seed(1)
    weight = torch.randn(17, 8, dtype=torch.float64)
    bias = torch.randn(17, dtype=torch.float64)
    _, _, db = oracle.dense_linear_ce_grads(hidden, weight, labels, bias=bias, reduction="sum")
    assert abs(float(db.sum())) < 1e-12
    # a saturated soft cap kills the gradient: |z| >> cap -> 1 - tanh^2 -> 0
    dh, dw, _ = oracle.dense_linear_ce_grads(hidden * 1e4, weight, labels, reduction="sum",
                                             logit_softcap=0.5)
    assert float(dh.abs().max()) < 1e-9 and float(dw.abs().max()) < 1e-6
    # lse >= max logit, and ignored rows contribute exactly nothing
    labels2 = labels.clone()
    labels2[1] = -100
    loss, lse = oracle.dense_linear_ce(hidden, weight, labels2, reduction="none", return_lse=True)
    assert float(loss[1]) == 0.0
    assert bool((lse >= (hidden @ weight.t()).max(dim=-1).values).all())
    dh, _, _ = oracle.dense_linear_ce_grads(hidden, weight, labels2, reduction="mean")
    assert torch.count_nonzero(dh[1]) == 0


@pytest.mark.parametrize("tile", [1, 5, 7, 64])
def test_online_tiled_algorithm_is_tile_invariant(tile):
    # tile sizes of test_tiled_linear_cross_entropy.py:172-219
    torch.manual_seed(31)
    hidden = torch.randn(15, 9, dtype=torch.float64)
    weight = torch.randn(23, 9, dtype=torch.float64)
    bias = torch.randn(23, dtype=torch.float64)
    labels = torch.randint(0, 22, (15,))
    labels[0] = -100
    logits = hidden @ weight.t() + bias
    logits[:, 22] = -float("inf")
    ref = F.cross_entropy(logits, labels, reduction="none", ignore_index=-100)
    losses, lse = oracle.online_tiled_linear_ce(hidden, weight, labels, vocab_block_size=tile,
                                                bias=bias, exclude_index=22, dtype=torch.float64)
    torch.testing.assert_close(losses, ref, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(lse, torch.logsumexp(logits, dim=-1), atol=1e-12, rtol=1e-12)


def test_rounded_logit_gradient_variant_stays_close_and_differs():
    torch.manual_seed(11)
    hidden = torch.randn(16, 32).bfloat16()
    weight = (torch.randn(200, 32) * 0.1).bfloat16()
    labels = torch.randint(0, 200, (16,))
    exact = oracle.dense_linear_ce_grads(hidden, weight, labels, reduction="mean")
    rounded = oracle.dense_linear_ce_grads(hidden, weight, labels, reduction="mean",
                                           round_grad_logits=torch.bfloat16)
    for a, e in zip(rounded[:2], exact[:2]):
        err = oracle.relative_max_error(a, e)
        assert 0.0 < err < 2e-2


def test_compaction_oracle_matches_nonzero_and_loop():
    rng = np.random.default_rng(5)
    for n in (0, 1, 63, 64, 65, 1000, 4097):
        labels = rng.integers(0, 50, size=n)
        labels[rng.random(n) < 0.4] = -100
        got = oracle.compact_rows(labels)
        assert got.dtype == np.int64
        ref = torch.nonzero(torch.from_numpy(labels) != -100).flatten().numpy()
        np.testing.assert_array_equal(got, ref)
        if n <= 1000:
            assert got.tolist() == oracle.compact_rows_loop(labels)
    assert oracle.compact_rows(np.full(10, -100)).size == 0
    np.testing.assert_array_equal(oracle.compact_rows(np.arange(10)), np.arange(10))


@pytest.mark.parametrize("splits", [(0, 13), (0, 5, 13), (0, 1, 6, 7, 13)])
@pytest.mark.parametrize("softcap,exclude", [(0.0, -1), (3.0, -1), (0.0, 6), (2.5, 0)])
def test_vocab_shard_statistics_combine_to_the_dense_loss(splits, softcap, exclude):
    """Any split of the vocabulary must combine to F.cross_entropy over the whole
    head (a library routine neither shard function calls).  A shard that holds
    only the excluded column (the [6,7) shard with exclude 6) has max -inf, sum 0."""
    torch.manual_seed(11)
    n, h, v = 9, 7, 13
    hidden = torch.randn(n, h, dtype=torch.float64)
    weight = torch.randn(v, h, dtype=torch.float64)
    bias = torch.randn(v, dtype=torch.float64)
    labels = torch.randint(0, v, (n,))
    labels[labels == exclude] = (exclude + 1) % v
    labels[2] = -100
    z = hidden @ weight.t() + bias
    if softcap:
        z = torch.tanh(z / softcap) * softcap
    if exclude >= 0:
        z[:, exclude] = -float("inf")
    expect = F.cross_entropy(z, labels, ignore_index=-100, reduction="none")
    stats = [
        oracle.vocab_shard_stats(hidden, weight[a:b], labels, vocab_start=a, bias=bias[a:b],
                                 exclude_index=exclude, logit_softcap=softcap)
        for a, b in zip(splits[:-1], splits[1:])
    ]
    losses, lse = oracle.combine_vocab_shards(stats, labels)
    torch.testing.assert_close(losses, expect, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(lse, torch.logsumexp(z, dim=1), rtol=1e-12, atol=1e-12)
    for s in stats:
        assert float(s[3]) == n - 1          # every shard counts every valid row
    if exclude == 6 and (6, 7) in list(zip(splits[:-1], splits[1:])):
        lonely = stats[list(zip(splits[:-1], splits[1:])).index((6, 7))]
        assert torch.isinf(lonely[0]).all() and (lonely[0] < 0).all()
        assert torch.count_nonzero(lonely[1]) == 0


def test_vocab_shard_statistics_brute_force_and_excluded_target():
    torch.manual_seed(12)
    n, h, v0, vl = 4, 3, 5, 6
    hidden = torch.randn(n, h, dtype=torch.float64)
    shard = torch.randn(vl, h, dtype=torch.float64)
    labels = torch.tensor([5, 7, 20, -100])      # first, inside (== exclude), other shard, ignored
    mx, sm, tg, cnt = oracle.vocab_shard_stats(hidden, shard, labels, vocab_start=v0,
                                               exclude_index=7)
    for r in range(n):
        zs = [sum(float(hidden[r, k]) * float(shard[c, k]) for k in range(h)) for c in range(vl)]
        kept = [z for c, z in enumerate(zs) if v0 + c != 7]
        assert math.isclose(float(mx[r]), max(kept), rel_tol=1e-12)
        assert math.isclose(float(sm[r]), sum(math.exp(z - max(kept)) for z in kept), rel_tol=1e-12)
    assert math.isclose(float(tg[0]), sum(float(hidden[0, k]) * float(shard[0, k]) for k in range(h)),
                        rel_tol=1e-12)
    assert float(tg[1]) == -math.inf             # label is the excluded column and local
    assert float(tg[2]) == 0.0 and float(tg[3]) == 0.0
    assert float(cnt) == 3.0


def test_label_on_the_excluded_column_gets_no_gradient_there():
    """Degenerate input the reference defines by construction: the excluded
    column is skipped before the onehot term (fused_linear_ce_cuda.cu:270-283),
    so a row labelled with it has gradient softmax(z) on the other columns and
    0 on the excluded one -- brute force on a 1 x 3 case."""
    hidden = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    weight = torch.tensor([[0.5, 0.25], [-1.0, 0.5], [2.0, 1.0]], dtype=torch.float64)
    labels = torch.tensor([1])
    dh, dw, _ = oracle.dense_linear_ce_grads(hidden, weight, labels, None, reduction="sum",
                                             exclude_index=1)
    z = [0.5 - 0.5, -1.0 - 1.0, 2.0 - 2.0]
    p0 = math.exp(z[0]) / (math.exp(z[0]) + math.exp(z[2]))
    g = [p0, 0.0, 1.0 - p0]
    for c in range(3):
        for k in range(2):
            assert math.isclose(float(dw[c, k]), g[c] * float(hidden[0, k]), abs_tol=1e-12)
    for k in range(2):
        assert math.isclose(float(dh[0, k]), sum(g[c] * float(weight[c, k]) for c in range(3)),
                            abs_tol=1e-12)


def test_soft_embedding_oracle_brute_force_and_limits():
    torch.manual_seed(21)
    hidden = torch.randn(3, 4, dtype=torch.float64)
    weight = torch.randn(5, 4, dtype=torch.float64)
    got = oracle.dense_soft_embedding(hidden, weight, logit_softcap=1.5, embedding_scale=2.0)
    for r in range(3):
        z = [1.5 * math.tanh(sum(float(hidden[r, k]) * float(weight[c, k]) for k in range(4)) / 1.5)
             for c in range(5)]
        total = sum(math.exp(x) for x in z)
        for k in range(4):
            expect = 2.0 * sum(math.exp(z[c]) / total * float(weight[c, k]) for c in range(5))
            assert math.isclose(float(got[r, k]), expect, rel_tol=1e-12, abs_tol=1e-12)
    # library routine, no cap
    lib = torch.softmax(hidden @ weight.t(), dim=-1) @ weight
    torch.testing.assert_close(oracle.dense_soft_embedding(hidden, weight), lib, rtol=1e-12,
                               atol=1e-12)
    # zero hidden -> uniform softmax -> mean of the weight rows
    mean = oracle.dense_soft_embedding(torch.zeros(1, 4, dtype=torch.float64), weight)
    torch.testing.assert_close(mean[0], weight.mean(dim=0), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("softcap", [None, 2.5])
def test_frozen_kl_oracle_matches_library_kl_div_and_autograd(softcap):
    """The reference's own host cases (tests/unit/kernels/test_dflash_kl.py:13-76,
    seeds 17 and 23) against F.kl_div / autograd, which the oracle does not call."""
    torch.manual_seed(17 if softcap is None else 23)
    dh = torch.randn(7, 5, dtype=torch.float64, requires_grad=True)
    th = torch.randn(7, 6, dtype=torch.float64)
    dw = torch.randn(11, 5, dtype=torch.float64)
    tw = torch.randn(11, 6, dtype=torch.float64)
    scale = torch.randn(7, dtype=torch.float64)
    zd, zt = F.linear(dh, dw), F.linear(th, tw)
    if softcap:
        zd, zt = softcap * torch.tanh(zd / softcap), softcap * torch.tanh(zt / softcap)
    expect = F.kl_div(F.log_softmax(zd, dim=-1), F.softmax(zt, dim=-1), reduction="none").sum(-1)
    grad = torch.autograd.grad((expect * scale).sum(), dh)[0]
    got = oracle.dense_frozen_kl(dh.detach(), dw, th, tw, logit_softcap=softcap)
    torch.testing.assert_close(got, expect.detach(), rtol=1e-12, atol=1e-12)
    got_grad = oracle.dense_frozen_kl_grad(dh.detach(), dw, th, tw, scale, logit_softcap=softcap)
    torch.testing.assert_close(got_grad, grad, rtol=1e-10, atol=1e-12)
    # same head on both sides: zero divergence, zero gradient
    same = oracle.dense_frozen_kl(dh.detach(), dw, dh.detach(), dw, logit_softcap=softcap)
    assert float(same.abs().max()) < 1e-12
    zero = oracle.dense_frozen_kl_grad(dh.detach(), dw, dh.detach(), dw, scale,
                                       logit_softcap=softcap)
    assert float(zero.abs().max()) < 1e-12
    assert bool((got >= 0).all())


@pytest.mark.parametrize("softcap,mult", [(None, 1.0), (2.0, 0.7)])
def test_ce_topk_oracle_matches_library_topk_and_autograd(softcap, mult):
    torch.manual_seed(41)
    n, h, v, k = 6, 5, 17, 4
    hidden = torch.randn(n, h, dtype=torch.float64, requires_grad=True)
    weight = torch.randn(v, h, dtype=torch.float64)
    labels = torch.randint(0, v, (n,))
    z = hidden @ weight.t() * mult
    if softcap:
        z = softcap * torch.tanh(z / softcap)
    loss = F.cross_entropy(z, labels, reduction="none")
    values, ids = z.topk(k, dim=-1)
    gl, gp, gv = torch.randn(n).double(), torch.randn(n).double(), torch.randn(n, k).double()
    objective = (gl * loss).sum() + (gp * torch.exp(-loss)).sum() + (gv * values).sum()
    grad = torch.autograd.grad(objective, hidden)[0]
    o_loss, o_prob, o_vals, o_ids, o_lse = oracle.dense_ce_topk(
        hidden.detach(), weight, labels, k, output_multiplier=mult, logit_softcap=softcap)
    torch.testing.assert_close(o_loss, loss.detach(), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(o_prob, torch.exp(-loss).detach(), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(o_vals, values.detach(), rtol=0, atol=0)
    assert torch.equal(o_ids, ids)
    torch.testing.assert_close(o_lse, torch.logsumexp(z, dim=-1).detach(), rtol=1e-12, atol=1e-12)
    o_grad = oracle.dense_ce_topk_grad(hidden.detach(), weight, labels, ids, gl, gp, gv,
                                       output_multiplier=mult, logit_softcap=softcap)
    torch.testing.assert_close(o_grad, grad, rtol=1e-10, atol=1e-12)


def test_ce_topk_oracle_orders_ties_by_id():
    hidden = torch.tensor([[1.0, 0.0]], dtype=torch.float64)
    weight = torch.tensor([[2.0, 0.0], [3.0, 1.0], [2.0, 5.0], [3.0, -1.0], [1.0, 0.0]],
                          dtype=torch.float64)
    _, _, vals, ids, _ = oracle.dense_ce_topk(hidden, weight, torch.tensor([0]), 4)
    assert ids.tolist() == [[1, 3, 0, 2]] and vals.tolist() == [[3.0, 3.0, 2.0, 2.0]]


def test_rounded_logit_gradient_brute_force():
    """round_grad_logits pinned exactly: every logit gradient is formed with
    Python floats, rounded element by element to bfloat16 (torch's scalar
    conversion, a routine the oracle does not use), and contracted by loops."""
    torch.manual_seed(12)
    n, h, v = 5, 4, 7
    hidden = torch.randn(n, h).bfloat16()
    weight = (torch.randn(v, h) * 0.5).bfloat16()
    labels = torch.tensor([3, -100, 0, 6, 2])
    valid = [y for y in labels.tolist() if y != -100]
    dh = [[0.0] * h for _ in range(n)]
    dw = [[0.0] * h for _ in range(v)]
    for r in range(n):
        y = int(labels[r])
        if y == -100:
            continue
        z = [sum(float(hidden[r, k]) * float(weight[c, k]) for k in range(h)) for c in range(v)]
        zmax = max(z)
        denom = sum(math.exp(x - zmax) for x in z)
        for c in range(v):
            g = (math.exp(z[c] - zmax) / denom - (1.0 if c == y else 0.0)) / len(valid)
            g = float(torch.tensor(g, dtype=torch.float64).to(torch.bfloat16))   # the rounding point
            for k in range(h):
                dh[r][k] += g * float(weight[c, k])
                dw[c][k] += g * float(hidden[r, k])
    got_dh, got_dw, _ = oracle.dense_linear_ce_grads(hidden, weight, labels, reduction="mean",
                                                     round_grad_logits=torch.bfloat16)
    torch.testing.assert_close(got_dh, torch.tensor(dh, dtype=torch.float64), atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(got_dw, torch.tensor(dw, dtype=torch.float64), atol=1e-12, rtol=1e-10)
    # rounding after the contraction instead (a wrong rounding point) is not the same thing
    exact = oracle.dense_linear_ce_grads(hidden, weight, labels, reduction="mean")
    assert not torch.equal(got_dh, exact[0].bfloat16().double())


@pytest.mark.parametrize("softcap", [None, 5.0])
def test_dim_first_head_matches_library_cross_entropy_and_autograd(softcap):
    """weight_dim_first=True pinned against F.cross_entropy(hidden @ weight) and
    autograd through it (the [H, V] head multiplies without a transpose)."""
    torch.manual_seed(13)
    n, h, v = 9, 6, 11
    hidden = torch.randn(n, h, dtype=torch.float64, requires_grad=True)
    weight = (torch.randn(h, v, dtype=torch.float64) * 0.7).requires_grad_(True)
    bias = torch.randn(v, dtype=torch.float64, requires_grad=True)
    labels = torch.randint(0, v, (n,))
    labels[2] = -100
    logits = hidden @ weight + bias
    if softcap:
        logits = torch.tanh(logits / softcap) * softcap
    ref = F.cross_entropy(logits, labels, ignore_index=-100, reduction="sum")
    ref.backward()
    got = oracle.dense_linear_ce(hidden.detach(), weight.detach(), labels, bias=bias.detach(),
                                 reduction="sum", logit_softcap=softcap, weight_dim_first=True)
    torch.testing.assert_close(got, ref.detach(), atol=1e-12, rtol=1e-12)
    dh, dw, db = oracle.dense_linear_ce_grads(hidden.detach(), weight.detach(), labels,
                                              bias=bias.detach(), reduction="sum",
                                              logit_softcap=softcap, weight_dim_first=True)
    assert dw.shape == weight.shape
    torch.testing.assert_close(dh, hidden.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(dw, weight.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(db, bias.grad, atol=1e-12, rtol=1e-10)


@pytest.mark.parametrize("multiplier,softcap,exclude", [(None, None, None), (0.25, None, 4),
                                                        (3.0, 8.0, None), (0.5, 6.0, 2)])
def test_masked_token_loss_oracle_matches_library_expression(multiplier, softcap, exclude):
    """The loss-method restatement against the sequence of library calls the
    reference makes (nemotron/model.py:2084-2151: scaled hidden states, logits,
    soft cap, -inf on the mask token, F.cross_entropy(reduction='none'), weights,
    / valid_token_count * scale) and autograd through it."""
    torch.manual_seed(14)
    n, h, v = 12, 5, 9
    hidden = torch.randn(n, h, dtype=torch.float64, requires_grad=True)
    weight = (torch.randn(v, h, dtype=torch.float64) * 0.6).requires_grad_(True)
    bias = torch.randn(v, dtype=torch.float64, requires_grad=True)
    labels = torch.randint(0, v, (n,))
    if exclude is not None:
        labels[labels == exclude] = (exclude + 1) % v
    labels[[1, 7]] = -100
    weights = torch.rand(n, dtype=torch.float64) + 0.1
    count, scale = 7.0, 2.0
    rows = torch.nonzero(labels != -100).flatten()
    active = hidden.index_select(0, rows)
    if multiplier is not None:
        active = active * multiplier
    logits = active @ weight.t() + bias
    if softcap:
        logits = torch.tanh(logits / softcap) * softcap
    if exclude is not None:
        logits = logits.clone()
        logits[:, exclude] = -float("inf")
    token_losses = F.cross_entropy(logits, labels[rows], ignore_index=-100, reduction="none")
    ref = (token_losses * weights[rows]).sum() / count * scale
    ref.backward()
    kw = dict(bias=bias.detach(), exclude_index=exclude, output_multiplier=multiplier,
              logit_softcap=softcap, loss_scale=scale)
    got = oracle.masked_token_loss(hidden.detach(), weight.detach(), labels, weights, count, **kw)
    torch.testing.assert_close(got, ref.detach(), atol=1e-12, rtol=1e-12)
    dh, dw, db = oracle.masked_token_loss_grads(hidden.detach(), weight.detach(), labels, weights,
                                                count, **kw)
    torch.testing.assert_close(dh, hidden.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(dw, weight.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(db, bias.grad, atol=1e-12, rtol=1e-10)
    assert torch.count_nonzero(dh[[1, 7]]) == 0


# ----------------------------------------------------------- DFlash loss method ----
def _dflash_case(seed, batch=3, tokens=7, h=6, ht=5, v=11, density=0.5):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(batch, tokens, h, generator=gen, dtype=torch.float64)
    teacher = torch.randn(batch, tokens, ht, generator=gen, dtype=torch.float64)
    draft_w = torch.randn(v, h, generator=gen, dtype=torch.float64) * 0.7
    teacher_w = torch.randn(v, ht, generator=gen, dtype=torch.float64) * 0.7
    targets = torch.randint(0, v, (batch, tokens), generator=gen)
    mask = torch.rand(batch, tokens, generator=gen) < density
    weights = torch.rand(batch, tokens, generator=gen, dtype=torch.float64) + 0.25
    counts = mask.sum(dim=1).to(torch.float64) + 1.0
    return hidden, teacher, draft_w, teacher_w, targets, mask, weights, counts


@pytest.mark.parametrize("loss_kind", ["paper_ce", "speculators_kl"])
@pytest.mark.parametrize("softcap", [None, 3.0])
def test_dflash_loss_oracle_matches_the_reference_call_sequence(loss_kind, softcap):
    """The sequence of library calls distributed_dflash_loss makes
    (dflash/model.py:870-955): nonzero, index_select, F.cross_entropy / F.kl_div
    on dense logits, scatter_add_, / (count + 1e-5), mean, * scale; gradients by
    autograd through it."""
    hidden, teacher, draft_w, teacher_w, targets, mask, weights, counts = _dflash_case(41)
    hidden = hidden.requires_grad_(True)
    draft_w = draft_w.requires_grad_(True)
    idx = torch.nonzero(mask.reshape(-1), as_tuple=False).flatten()
    rows = hidden.reshape(-1, hidden.shape[-1]).index_select(0, idx)
    pw = weights.reshape(-1).index_select(0, idx)

    def capped(z):
        return z if softcap is None else softcap * torch.tanh(z / softcap)
    draft_logits = capped(F.linear(rows, draft_w))
    if loss_kind == "paper_ce":
        token_loss = F.cross_entropy(draft_logits, targets.reshape(-1).index_select(0, idx),
                                     reduction="none")
    else:
        trows = teacher.reshape(-1, teacher.shape[-1]).index_select(0, idx)
        teacher_logits = capped(F.linear(trows, teacher_w))
        token_loss = F.kl_div(F.log_softmax(draft_logits, dim=-1),
                              F.softmax(teacher_logits, dim=-1), reduction="none").sum(dim=-1)
    numerators = torch.zeros(mask.shape[0], dtype=torch.float64)
    numerators.scatter_add_(0, torch.div(idx, mask.shape[1], rounding_mode="floor"),
                            token_loss * pw)
    expect = (numerators / (counts + 1.0e-5)).mean() * 1.75
    expect.backward()

    kw = dict(loss_kind=loss_kind, teacher_hidden_states=teacher, teacher_weight=teacher_w,
              logit_softcap=softcap, loss_scale=1.75)
    got = oracle.dflash_token_loss(hidden.detach(), targets, mask, weights, draft_w.detach(),
                                   counts, **kw)
    torch.testing.assert_close(got, expect.detach(), rtol=1e-12, atol=1e-12)
    dh, dw = oracle.dflash_token_loss_grads(hidden.detach(), targets, mask, weights,
                                            draft_w.detach(), counts, **kw)
    torch.testing.assert_close(dh, hidden.grad, rtol=1e-10, atol=1e-12)
    assert torch.count_nonzero(dh.reshape(-1, dh.shape[-1])[~mask.reshape(-1)]) == 0
    if loss_kind == "paper_ce":
        torch.testing.assert_close(dw, draft_w.grad, rtol=1e-10, atol=1e-12)
    else:
        assert dw is None


def test_dflash_loss_oracle_per_sample_loop_and_empty_batch():
    hidden, teacher, draft_w, teacher_w, targets, mask, weights, counts = _dflash_case(43)
    mask[1] = False                       # a sample without supervised positions
    batch, tokens = mask.shape
    total = 0.0
    for b in range(batch):                # brute force, one sample and one position at a time
        num = 0.0
        for t in range(tokens):
            if not bool(mask[b, t]):
                continue
            z = [float(hidden[b, t] @ draft_w[v]) for v in range(draft_w.shape[0])]
            lse = math.log(sum(math.exp(x) for x in z))
            num += (lse - z[int(targets[b, t])]) * float(weights[b, t])
        total += num / (float(counts[b]) + 1.0e-5)
    got = oracle.dflash_token_loss(hidden, targets, mask, weights, draft_w, counts,
                                   loss_kind="paper_ce")
    assert abs(float(got) - total / batch) <= 1e-12 * abs(total)
    # the scatter-add on its own
    idx = torch.nonzero(mask.reshape(-1)).flatten()
    vals = torch.arange(1, idx.numel() + 1, dtype=torch.float64)
    w = weights.reshape(-1)[idx]
    expect = torch.zeros(batch, dtype=torch.float64).scatter_add_(0, idx // tokens, vals * w)
    torch.testing.assert_close(oracle.segment_weighted_sum(vals, w, idx, tokens, batch), expect)
    assert float(oracle.segment_weighted_sum(vals, None, idx, tokens, batch)[1]) == 0.0
    # nothing supervised: exactly zero, zero gradient
    none = torch.zeros_like(mask)
    assert float(oracle.dflash_token_loss(hidden, targets, none, weights, draft_w, counts,
                                          loss_kind="paper_ce")) == 0.0
    dh, dw = oracle.dflash_token_loss_grads(hidden, targets, none, weights, draft_w, counts,
                                            loss_kind="paper_ce")
    assert torch.count_nonzero(dh) == 0 and dw is None
    with pytest.raises(ValueError):
        oracle.dflash_token_loss(hidden, targets, mask, weights, draft_w, counts, loss_kind="kl")


def test_masked_token_loss_oracle_rounding_point_of_the_scaled_hidden_states():
    """round_scaled_hidden=True rounds hidden * multiplier to the 16-bit dtype before the
    projection, the order of the reference's loss method (nemotron/model.py:2084-2086):
    pinned against the library expression on the rounded product."""
    gen = torch.Generator().manual_seed(5)
    hidden = torch.randn(9, 16, generator=gen).bfloat16()
    weight = (torch.randn(23, 16, generator=gen) * 0.3).bfloat16()
    labels = torch.randint(0, 23, (9,), generator=gen)
    labels[2] = -100
    weights = torch.rand(9, generator=gen) + 0.5
    scaled = (hidden * 1.75)                      # bf16 tensor times a Python float: rounds to bf16
    assert scaled.dtype == torch.bfloat16
    logits = F.linear(scaled.double(), weight.double())
    token = F.cross_entropy(logits, labels, reduction="none", ignore_index=-100)
    expect = (token * weights.double()).sum() / 8.0
    got = oracle.masked_token_loss(hidden, weight, labels, weights, 8.0, output_multiplier=1.75,
                                   round_scaled_hidden=True)
    torch.testing.assert_close(got, expect, rtol=1e-12, atol=1e-12)
    plain = oracle.masked_token_loss(hidden, weight, labels, weights, 8.0, output_multiplier=1.75)
    assert float(plain) != float(got) and abs(float(plain) - float(got)) < 1e-2 * float(got)
    # a power of two rounds nothing
    a = oracle.masked_token_loss(hidden, weight, labels, weights, 8.0, output_multiplier=0.5)
    b = oracle.masked_token_loss(hidden, weight, labels, weights, 8.0, output_multiplier=0.5,
                                 round_scaled_hidden=True)
    assert float(a) == float(b)
