"""Construction-time environment switches of the expert path.

The names are the reference's own, so a launcher that already exports them
(scripts/lib/speed_stack.sh:13-35 in the reference) drives this implementation
unchanged.  Modules read them once in ``__init__`` and keep the value as an
attribute; nothing reads the environment inside a forward.
"""

from __future__ import annotations

import os

import torch

from nestor_amd import _lib


def _is_one(name: str, default: str = "0") -> bool:
    return os.environ.get(name, default) == "1"


def stacked_banks_requested() -> bool:
    """``NESTOR_STACKED_EXPERT_BANKS=1`` (nestor/backbones/expert_bank_stack.py:52-55)."""

    return _is_one("NESTOR_STACKED_EXPERT_BANKS")


def fused_gate_requested() -> bool:
    """``NESTOR_GROUPED_MM_FUSED_GATE=1`` (nestor/backbones/grouped_mm.py:180-194)."""

    return _is_one("NESTOR_GROUPED_MM_FUSED_GATE")


def triton_index_requested() -> bool:
    """``NESTOR_TRITON_INDEX_BUILD=1`` (nestor/backbones/triton_dispatch.py:49-60);
    here it selects the HIP index build."""

    return _is_one("NESTOR_TRITON_INDEX_BUILD")


def triton_expert_requested() -> bool:
    """``NESTOR_TRITON_EXPERT_DISPATCH``, defaulting to the index-build flag
    (nestor/backbones/triton_expert.py:80-95); here it selects the fused HIP path."""

    value = os.environ.get("NESTOR_TRITON_EXPERT_DISPATCH")
    if value is None:
        value = os.environ.get("NESTOR_TRITON_INDEX_BUILD", "0")
    return value == "1"


def triton_cat_cast_requested() -> bool:
    """``NESTOR_TRITON_EXPERT_CATCAST`` (default on; triton_expert.py:98-109)."""

    return _is_one("NESTOR_TRITON_EXPERT_CATCAST", "1")


def batched_routers_enabled() -> bool:
    """``NESTOR_BATCHED_ROUTERS=1`` (nestor/backbones/batched_router.py:50-57)."""

    return _is_one("NESTOR_BATCHED_ROUTERS")


def pool_grouped_mm_disabled() -> bool:
    """``NESTOR_POOL_GROUPED_MM=0`` opt-out (nestor/backbones/expert_pools.py:345-349)."""

    return os.environ.get("NESTOR_POOL_GROUPED_MM", "1") == "0"


def hip_available() -> bool:
    """Whether the HIP kernels can run: the library is built and a GPU is visible."""

    return _lib.library_available() and torch.cuda.is_available()


# The reference spells availability per feature; all three mean the same here.
triton_index_available = hip_available
triton_expert_available = hip_available
