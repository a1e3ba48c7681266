"""nestor_amd: MI355X-native (gfx950) kernels for Nestor's routed hybrid
expert-MLP path, behind the reference's own Python entry points."""

from nestor_amd.bank import (
    StackedBanksMixin,
    StackedExpertBank,
    SwigluExpert,
    consolidate_stacked_expert_banks,
)
from nestor_amd.dispatch import DispatchPlan, build_dispatch_maps, dispatch_plan
from nestor_amd.expert_kernels import (
    bank_is_fusable,
    cat_cast,
    combine_rows,
    dispatch_rows,
    gate_combine_slots,
    pack_rows,
    swiglu,
    swiglu_fused,
)
from nestor_amd.grouped import (
    GROUPED_MM_ALIGN,
    autocast_dtype,
    grouped_expert_combine,
    grouped_expert_rows,
    segment_mm,
)
from nestor_amd.pool import ExpertPoolMLP
from nestor_amd.router import Router, RouterOutput, route_private_batched

__all__ = [
    "DispatchPlan", "ExpertPoolMLP", "GROUPED_MM_ALIGN", "Router", "RouterOutput",
    "StackedBanksMixin", "StackedExpertBank", "SwigluExpert", "autocast_dtype",
    "bank_is_fusable", "build_dispatch_maps", "cat_cast", "combine_rows",
    "consolidate_stacked_expert_banks", "dispatch_plan", "dispatch_rows", "gate_combine_slots",
    "grouped_expert_combine", "grouped_expert_rows", "pack_rows", "route_private_batched",
    "segment_mm",
    "swiglu", "swiglu_fused",
]
