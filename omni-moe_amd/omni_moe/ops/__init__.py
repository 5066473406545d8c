"""Operators of the OmniMoE forward path (HIP kernels for MI355X)."""
from .hip import (  # noqa: F401
    hip_omni_expert_func,
    hip_omni_mlp_func,
    hip_omni_router_func,
    hip_omni_router_fwd_func,
    hip_omni_schedule_func,
)
