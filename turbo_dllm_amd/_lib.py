"""ctypes binding of libtlce_gfx950.so (declarations: include/tlce.h).

Takes the place of the reference's native-extension resolver
(dllm_parallel/core/kernels/chunked_linear_ce_native.py:35-46 and
dllm_parallel/core/kernels/runtime.py:189-223): one cached handle, required
symbols checked at load, and a hard failure -- never a silent fallback -- when
the library has not been built.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_void_p, POINTER
from functools import lru_cache
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
LIBRARY_PATH = PACKAGE_DIR / "libtlce_gfx950.so"

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
REDUCTION_NONE, REDUCTION_SUM, REDUCTION_MEAN = 0, 1, 2

# name -> (restype, argtypes); mirrors include/tlce.h one to one
SIGNATURES = {
    "tlce_version": (c_int, []),
    "tlce_last_error": (c_char_p, []),
    "tlce_check_device": (c_int, [c_int]),
    "tlce_compact_workspace_bytes": (c_int64, [c_int64]),
    "tlce_compact_rows": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p],
    ),
    "tlce_compact_mask": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p],
    ),
    "tlce_gather_rows": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "tlce_scatter_rows": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "tlce_fill_zero": (c_int, [c_void_p, c_int64, c_void_p]),
    "tlce_gather_loss_rows": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden labels weights row_idx count
            c_int64, c_int64, c_int64, c_int64,                 # capacity padded_rows row_bytes ignore
            c_void_p, c_void_p, c_void_p, c_void_p,             # hidden_dst labels_dst weights_dst stream
        ],
    ),
    "tlce_forward_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int]),
    "tlce_forward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels row_idx
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int64, c_int64, c_float,                          # ignore exclude softcap
            c_void_p, c_void_p, c_void_p,                       # losses lse valid_count
            c_void_p, c_int64, c_void_p,                        # workspace bytes stream
        ],
    ),
    "tlce_forward_noalloc": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels row_idx
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int64, c_int64, c_float,                          # ignore exclude softcap
            c_void_p, c_void_p, c_void_p,                       # losses lse valid_count
            c_void_p,                                           # stream
        ],
    ),
    "tlce_backward_workspace_bytes": (
        c_int64,
        [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int64],
    ),
    "tlce_backward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels row_idx
            c_void_p, c_void_p, c_void_p,                       # lse valid_count grad_output
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int, c_int64, c_int64, c_float,                   # reduction ignore exclude softcap
            c_void_p, c_void_p, c_void_p,                       # grad_hidden grad_weight grad_bias
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_dim_first_supported": (c_int, [c_int64, c_int64, c_int]),
    "tlce_forward_dim_first": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels row_idx
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int64, c_int64, c_float,                          # ignore exclude softcap
            c_void_p, c_void_p, c_void_p,                       # losses lse valid_count
            c_void_p, c_int64, c_void_p,                        # workspace bytes stream
        ],
    ),
    "tlce_backward_dim_first": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels row_idx
            c_void_p, c_void_p, c_void_p,                       # lse valid_count grad_output
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int, c_int64, c_int64, c_float,                   # reduction ignore exclude softcap
            c_void_p, c_void_p, c_void_p,                       # grad_hidden grad_weight grad_bias
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_fused_gradients_supported": (c_int, [c_int64, c_int64, c_int]),
    "tlce_query_fused_plan": (
        c_int, [c_int64, c_int64, c_int64, c_int, c_int64, c_void_p, c_void_p, c_void_p]
    ),
    "tlce_forward_with_gradients_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int, c_int, c_int64]
    ),
    "tlce_forward_with_gradients": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight labels row_idx weights
            c_void_p,                                           # row_count
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int64, c_int64, c_float, c_float,                 # ignore exclude softcap multiplier
            c_void_p, c_void_p, c_void_p,                       # losses lse valid_count
            c_void_p, c_void_p,                                 # grad_hidden_f32 grad_weight_f32
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_ce_topk_gradient_in_forward_supported": (c_int, [c_int64, c_int64, c_int64, c_int]),
    "tlce_ce_topk_forward_with_gradient_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int, c_int64]),
    "tlce_ce_topk_forward_with_gradient": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int,  # h w labels m h v dtype k
            c_float, c_float,                                   # multiplier softcap
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # losses probs top_values top_ids lse
            c_void_p, c_int64, c_void_p, c_int64, c_void_p,     # unit panel_bytes ws bytes stream
        ],
    ),
    "tlce_ce_topk_apply_gradient": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # unit hidden weight labels top_ids
            c_void_p, c_void_p,                                 # ce_scale grad_top_values
            c_int64, c_int64, c_int64, c_int, c_int,            # m h v dtype k
            c_float, c_float, c_void_p, c_void_p,               # multiplier softcap grad_hidden stream
        ],
    ),
    "tlce_grad_weight_from_panel": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p,                       # hidden row_idx row_count
            c_void_p, c_void_p,                                 # grad_output valid_count
            c_int64, c_int64, c_int64, c_int, c_int,            # m h v dtype reduction
            c_void_p, c_int64, c_void_p, c_int64, c_void_p,     # grad_weight panel_bytes ws bytes stream
        ],
    ),
    "tlce_apply_grad_output": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # dh32 dw32 row_idx row_count
            c_void_p, c_void_p,                                 # grad_output valid_count
            c_int64, c_int64, c_int64, c_int64, c_int, c_int,   # m n_out h v dtype reduction
            c_void_p, c_void_p, c_void_p,                       # grad_hidden grad_weight stream
        ],
    ),
    "tlce_masked_loss_forward_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int, c_int]
    ),
    "tlce_masked_loss_forward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels weights
            c_void_p, c_void_p,                                 # row_idx row_count
            c_int64, c_int64, c_int64, c_int64, c_int,          # m n_out h v dtype
            c_int64, c_int64, c_float, c_float,                 # ignore exclude softcap multiplier
            c_void_p, c_void_p, c_void_p, c_void_p,             # losses lse valid_count weighted_sum
            c_void_p, c_int64, c_void_p,                        # workspace bytes stream
        ],
    ),
    "tlce_masked_loss_backward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # hidden weight bias labels weights
            c_void_p, c_void_p,                                 # row_idx row_count
            c_void_p, c_void_p, c_void_p,                       # lse valid_count grad_output
            c_int64, c_int64, c_int64, c_int64, c_int, c_int,   # m n_out h v dtype reduction
            c_int64, c_int64, c_float, c_float,                 # ignore exclude softcap multiplier
            c_void_p, c_void_p, c_void_p,                       # grad_hidden grad_weight grad_bias
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_forward_local": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # hidden weight bias labels
            c_int64, c_int64, c_int64, c_int, c_int64,          # m h v_local dtype vocab_start
            c_int64, c_int64, c_float,                          # ignore exclude softcap
            c_void_p, c_void_p, c_void_p, c_void_p,             # local_max local_sum target count
            c_void_p, c_int64, c_void_p,                        # workspace bytes stream
        ],
    ),
    "tlce_backward_local": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # hidden weight bias labels
            c_void_p, c_void_p, c_void_p,                       # global_lse valid_count grad_output
            c_int64, c_int64, c_int64, c_int,                   # m h v_local dtype
            c_int, c_int64, c_int64, c_int64, c_float,          # reduction start ignore exclude cap
            c_void_p, c_void_p, c_void_p,                       # grad_hidden grad_weight grad_bias
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_soft_embedding_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int, c_int64]
    ),
    "tlce_soft_embedding": (
        c_int,
        [
            c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int,   # hidden weight m h v dtype
            c_float, c_float, c_void_p,                             # softcap scale out
            c_int64, c_void_p, c_int64, c_void_p,                   # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_kl_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int64, c_int, c_int64]
    ),
    "tlce_kl_forward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # draft h/w, teacher h/w
            c_int64, c_int64, c_int64, c_int64, c_int,          # m h_draft h_teacher v dtype
            c_float, c_void_p, c_void_p, c_void_p,              # softcap losses draft_lse teacher_lse
            c_void_p,                                           # teacher_probabilities (or null)
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_kl_gradient_in_forward_supported": (
        c_int, [c_int64, c_int64, c_int64, c_int64, c_int, c_float]),
    "tlce_kl_forward_with_gradient_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int64, c_int, c_int64]),
    "tlce_kl_forward_with_gradient": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # draft h/w, teacher h/w
            c_int64, c_int64, c_int64, c_int64, c_int,          # m h_draft h_teacher v dtype
            c_float, c_void_p, c_void_p, c_void_p,              # softcap losses draft_lse teacher_lse
            c_void_p,                                           # unit_grad_hidden_f32
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_kl_teacher_probabilities_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "tlce_kl_backward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # draft h/w, teacher h/w
            c_void_p, c_void_p, c_void_p,                       # draft_lse teacher_lse grad_output
            c_void_p,                                           # teacher_probabilities (or null)
            c_int64, c_int64, c_int64, c_int64, c_int,          # m h_draft h_teacher v dtype
            c_float, c_void_p,                                  # softcap grad_hidden
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_ce_topk_forward_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int, c_int64]
    ),
    "tlce_ce_topk_backward_workspace_bytes": (
        c_int64, [c_int64, c_int64, c_int64, c_int, c_int64]
    ),
    "tlce_ce_topk_forward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p,                       # hidden weight labels
            c_int64, c_int64, c_int64, c_int, c_int,            # m h v dtype top_k
            c_float, c_float,                                   # multiplier softcap
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # losses probs top_values top_ids lse
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_ce_topk_backward": (
        c_int,
        [
            c_void_p, c_void_p, c_void_p, c_void_p,             # hidden weight labels lse
            c_void_p, c_void_p, c_void_p,                       # top_ids ce_scale grad_top_values
            c_int64, c_int64, c_int64, c_int, c_int,            # m h v dtype top_k
            c_float, c_float, c_void_p,                         # multiplier softcap grad_hidden
            c_int64, c_void_p, c_int64, c_void_p,               # panel_bytes workspace bytes stream
        ],
    ),
    "tlce_segment_weighted_sum": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p],
    ),
    "tlce_profile_begin": (c_int, []),
    "tlce_profile_end": (c_int, [c_void_p, c_void_p, c_int]),
    "tlce_query_plan": (
        c_int,
        [
            c_int64, c_int64, c_int64, c_int, c_int, c_int64,
            POINTER(c_int), POINTER(c_int64), POINTER(c_int64),
            POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
        ],
    ),
}


class NativeLibraryMissing(RuntimeError):
    pass


@lru_cache(maxsize=1)
def library() -> ctypes.CDLL:
    """Loads the HIP library once; raises if it is absent or incomplete."""
    if not LIBRARY_PATH.exists():
        raise NativeLibraryMissing(
            f"{LIBRARY_PATH} is missing: the gfx950 HIP library has not been built. "
            "Run `python -m turbo_dllm_amd.build` (or __graft_entry__.build()). "
            "Device tensors are never routed to a CPU or PyTorch fallback."
        )
    # torch ships its own HIP runtime.  Loading it first makes this library bind
    # to that same runtime; two runtimes in one process do not share the GPU.
    import torch  # noqa: F401

    lib = ctypes.CDLL(str(LIBRARY_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise NativeLibraryMissing(
                f"{LIBRARY_PATH} does not export {name!r}; rebuild the library"
            ) from exc
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def last_error() -> str:
    message = library().tlce_last_error()
    return message.decode("utf-8", "replace") if message else ""


def check(code: int, what: str) -> None:
    """Raises RuntimeError with the library's message when a call failed."""
    if code != 0:
        raise RuntimeError(f"{what} failed: {last_error()}")


def query_plan(m: int, h: int, v: int, dtype_code: int, compute_weight_grad: bool,
               panel_bytes: int = 0) -> dict:
    """Tile plan the host scheduler would use (no GPU needed)."""
    engine = c_int()
    tile, splits, columns, panels, ksplits = (c_int64() for _ in range(5))
    check(
        library().tlce_query_plan(
            m, h, v, dtype_code, int(compute_weight_grad), panel_bytes,
            ctypes.byref(engine), ctypes.byref(tile), ctypes.byref(splits),
            ctypes.byref(columns), ctypes.byref(panels), ctypes.byref(ksplits),
        ),
        "tlce_query_plan",
    )
    return {
        "engine": {0: "generic", 1: "mfma", 2: "mfma_direct"}[engine.value],
        "tile": tile.value,
        "forward_vocab_splits": splits.value,
        "panel_columns": columns.value,
        "n_panels": panels.value,
        "grad_hidden_k_splits": ksplits.value,
    }


def query_fused_plan(m: int, h: int, v: int, dtype_code: int, panel_bytes: int = 0) -> dict:
    """How the forward that leaves the gradients would take ``m`` rows: rows per
    block, blocks, and K splits of the grad_hidden contraction (no GPU needed)."""
    block_rows = c_int64()
    n_blocks, ksplits = c_int(), c_int()
    check(
        library().tlce_query_fused_plan(
            m, h, v, dtype_code, panel_bytes, ctypes.byref(block_rows), ctypes.byref(n_blocks),
            ctypes.byref(ksplits),
        ),
        "tlce_query_fused_plan",
    )
    return {"block_rows": block_rows.value, "n_blocks": n_blocks.value,
            "grad_hidden_k_splits": ksplits.value}


PROFILE_CLASSES = (
    "forward_stats", "combine_loss", "grad_logits_panel", "grad_hidden_gemm",
    "grad_weight_gemm", "transpose", "other", "exp_logits_panel",
)


class kernel_profile:
    """Context manager: per-kernel-class milliseconds and launch counts of the
    library calls made inside it (HIP events on the caller's stream)."""

    def __enter__(self):
        check(library().tlce_profile_begin(), "tlce_profile_begin")
        self.ms = {}
        self.launches = {}
        return self

    def __exit__(self, *exc):
        n = len(PROFILE_CLASSES)
        ms = (c_double * n)()
        counts = (c_int64 * n)()
        code = library().tlce_profile_end(ms, counts, n)
        if exc[0] is None:
            check(code, "tlce_profile_end")
        self.ms = dict(zip(PROFILE_CLASSES, (float(x) for x in ms)))
        self.launches = dict(zip(PROFILE_CLASSES, (int(x) for x in counts)))
        return False
