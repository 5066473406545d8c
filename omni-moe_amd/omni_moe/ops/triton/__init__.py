"""Import-path compatibility with the reference: ``from omni_moe.ops.triton import
triton_omni_mlp_func, triton_omni_router_func, triton_omni_expert_func``
(reference omni_moe/ops/triton/__init__.py:1-11).  No Triton is involved: the three names
are the HIP operators, which keep the reference's call signatures and, like them, are differentiable."""
from ..hip import hip_omni_expert_func as triton_omni_expert_func
from ..hip import hip_omni_mlp_func as triton_omni_mlp_func
from ..hip import hip_omni_router_func as triton_omni_router_func

__all__ = ["triton_omni_mlp_func", "triton_omni_router_func", "triton_omni_expert_func"]
