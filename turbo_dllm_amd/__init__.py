"""MI355X (gfx950) fused linear cross-entropy: the LM-head projection plus
masked-token loss behind the reference's loss API.

Package-level exports are lightweight proxies, as in the reference's
``dllm_parallel.core.kernels`` (dllm_parallel/core/kernels/__init__.py:34-39):
importing this package initialises neither torch nor the HIP library.
"""

from __future__ import annotations

import importlib
from typing import Any

__all__ = [
    "VocabParallelLinear",
    "chunked_linear_ce_native",
    "compact_valid_loss_rows",
    "dflash_token_loss",
    "frozen_linear_ce_topk",
    "frozen_linear_kl",
    "masked_token_loss",
    "tiled_linear_cross_entropy",
]

_SUBMODULES = {"chunked_linear_ce_native", "compaction", "layers", "loss", "build", "options",
               "dflash_kl", "dflash_linear_topk", "streaming_soft_embedding"}


def tiled_linear_cross_entropy(*args: Any, **kwargs: Any) -> Any:
    from .tiled_linear_cross_entropy import tiled_linear_cross_entropy as impl

    return impl(*args, **kwargs)


def compact_valid_loss_rows(*args: Any, **kwargs: Any) -> Any:
    from .compaction import compact_valid_loss_rows as impl

    return impl(*args, **kwargs)


def masked_token_loss(*args: Any, **kwargs: Any) -> Any:
    from .loss import masked_token_loss as impl

    return impl(*args, **kwargs)


def dflash_token_loss(*args: Any, **kwargs: Any) -> Any:
    from .loss import dflash_token_loss as impl

    return impl(*args, **kwargs)


def frozen_linear_ce_topk(*args: Any, **kwargs: Any) -> Any:
    from .dflash_linear_topk import frozen_linear_ce_topk as impl

    return impl(*args, **kwargs)


def frozen_linear_kl(*args: Any, **kwargs: Any) -> Any:
    from .dflash_kl import frozen_linear_kl as impl

    return impl(*args, **kwargs)


def __getattr__(name: str) -> Any:
    if name in _SUBMODULES:
        return importlib.import_module(f"{__name__}.{name}")
    if name == "VocabParallelLinear":
        from .layers import VocabParallelLinear

        return VocabParallelLinear
    raise AttributeError(name)
