"""Writes tests/golden/linear_ce_cases.npz: small seeded inputs with expected
losses and gradients.

The expected values do not come from the oracle or from the product: they are
produced by library routines only -- ``torch.nn.functional.cross_entropy`` on
dense float64 logits and torch autograd through it -- which is the same
closed form the reference's own tests compare against
(tests/unit/kernels/test_tiled_linear_cross_entropy.py:33-58).  The reference
holds no stored vectors for this path, so these fixtures are the stored form
of its seeded cases (same seeds, shapes and masks as :61-453 of that file)
plus a few extra shapes.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""

from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F

OUT = Path(__file__).resolve().parent / "linear_ce_cases.npz"

# name, seed, rows shape, H, V, options
CASES = [
    dict(name="ref_seed0_bias", seed=0, shape=(2, 5), h=7, v=13, bias=True, ignore=[(0, 1)]),
    dict(name="ref_seed2_exclude", seed=2, shape=(2, 3), h=5, v=11, exclude=10, label_hi=10),
    dict(name="ref_seed31_tiles", seed=31, shape=(3, 5), h=9, v=23, bias=True, exclude=22,
         label_hi=22, ignore=[(0, 0), (2, 4)]),
    dict(name="softcap_exclude", seed=7, shape=(6,), h=16, v=37, softcap=5.0, exclude=4,
         label_lo=5, ignore=[(2,)], hidden_scale=3.0),
    dict(name="softcap_bias", seed=8, shape=(4, 3), h=8, v=29, softcap=2.0, bias=True,
         hidden_scale=2.0),
    dict(name="wide_vocab", seed=9, shape=(5,), h=12, v=1031, ignore=[(1,), (3,)]),
]


def build(case):
    torch.manual_seed(case["seed"])
    shape, h, v = case["shape"], case["h"], case["v"]
    hidden = torch.randn(*shape, h, dtype=torch.float64) * case.get("hidden_scale", 1.0)
    weight = torch.randn(v, h, dtype=torch.float64)
    bias = torch.randn(v, dtype=torch.float64) if case.get("bias") else None
    labels = torch.randint(case.get("label_lo", 0), case.get("label_hi", v), shape)
    for pos in case.get("ignore", []):
        labels[pos] = -100
    grad_out = torch.randn(*shape, dtype=torch.float64)
    out = {"hidden": hidden, "weight": weight, "labels": labels, "grad_out": grad_out}
    if bias is not None:
        out["bias"] = bias
    for reduction in ("none", "sum", "mean"):
        hh = hidden.clone().requires_grad_(True)
        ww = weight.clone().requires_grad_(True)
        bb = bias.clone().requires_grad_(True) if bias is not None else None
        logits = hh.reshape(-1, h) @ ww.t()
        if bb is not None:
            logits = logits + bb
        if case.get("softcap"):
            logits = torch.tanh(logits / case["softcap"]) * case["softcap"]
        if case.get("exclude") is not None:
            mask = torch.zeros(v, dtype=torch.float64)
            mask[case["exclude"]] = -float("inf")
            logits = logits + mask
        loss = F.cross_entropy(logits, labels.reshape(-1), reduction=reduction, ignore_index=-100)
        if reduction == "none":
            loss = loss.reshape(shape)
            loss.backward(grad_out)
        else:
            loss.backward()
        out[f"loss_{reduction}"] = loss.detach()
        out[f"dh_{reduction}"] = hh.grad
        out[f"dw_{reduction}"] = ww.grad
        if bb is not None:
            out[f"db_{reduction}"] = bb.grad
    return out


def main():
    arrays = {}
    meta = []
    for case in CASES:
        for key, value in build(case).items():
            arrays[f"{case['name']}/{key}"] = value.numpy()
        meta.append(
            f"{case['name']}|softcap={case.get('softcap', 0)}|exclude={case.get('exclude', -1)}"
        )
    arrays["__cases__"] = np.array(meta)
    np.savez_compressed(OUT, **arrays)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(CASES)} cases)")


if __name__ == "__main__":
    main()
