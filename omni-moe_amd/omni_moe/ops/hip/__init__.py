from .interface import (  # noqa: F401
    Schedule,
    hip_omni_expert_func,
    hip_omni_router_func,
    hip_omni_schedule_func,
)

__all__ = ["hip_omni_router_func", "hip_omni_expert_func", "hip_omni_schedule_func", "Schedule"]
