from .interface import (  # noqa: F401
    Schedule,
    hip_add_inplace_func,
    hip_linear_func,
    hip_omni_expert_func,
    hip_omni_mlp_func,
    hip_omni_moe_fwd_func,
    hip_omni_router_func,
    hip_omni_router_fwd_func,
    hip_omni_schedule_func,
    hip_swiglu_linear_func,
)

__all__ = ["hip_omni_router_func", "hip_omni_expert_func", "hip_omni_mlp_func", "hip_omni_schedule_func",
           "hip_omni_router_fwd_func", "hip_linear_func", "hip_omni_moe_fwd_func", "hip_add_inplace_func", "hip_swiglu_linear_func", "Schedule"]
