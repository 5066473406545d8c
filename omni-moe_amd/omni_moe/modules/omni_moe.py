"""OmniMoE layer: drop-in for the reference's ``omni_moe.modules.omni_moe`` (forward path).

Same constructor, attribute / ``state_dict`` names and ``forward(hidden_states, **kwargs)``
as the reference's ``OmniMoE`` (omni_moe/modules/omni_moe.py:14-106); the forward runs three
calls into the gfx950 library: router (projection, BatchNorm, log-softmax, Cartesian top-k,
exp), fused atomic experts, and the shared SwiGLU MLP whose down projection adds the expert
output.  Forward only: outputs carry no autograd graph.
"""
import math

import torch
import torch.nn as nn

from omni_moe.ops.hip import (hip_linear_func, hip_omni_expert_func, hip_omni_mlp_func, hip_omni_router_fwd_func,
                              hip_swiglu_linear_func)


class OmniMoEConfig:
    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        hidden_act: str,
        num_experts: int,
        num_experts_per_token: int,
    ):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.hidden_act = hidden_act
        self.num_experts = num_experts
        self.num_experts_per_token = num_experts_per_token


class OmniMoE(nn.Module):
    def __init__(self, config: OmniMoEConfig):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        # the reference's kernels hard-wire silu whatever hidden_act says
        # (omni_expert.py:156, omni_mlp.py:60); anything else cannot be honoured
        if config.hidden_act not in ("silu", "swish"):
            raise ValueError(f"hidden_act={config.hidden_act!r}: the OmniMoE kernels implement silu only")
        self.hidden_act = config.hidden_act

        self.num_experts = config.num_experts
        self.num_expert_sqrt = math.floor(math.sqrt(self.num_experts))
        self.top_k = config.num_experts_per_token

        # shared expert
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=False)

        # router gate for retrieval experts
        self.router_gate_x = nn.Linear(self.hidden_size, self.num_expert_sqrt, bias=False)
        self.router_gate_y = nn.Linear(self.hidden_size, self.num_expert_sqrt, bias=False)
        self.router_norm_x = nn.BatchNorm1d(self.num_expert_sqrt, affine=False)
        self.router_norm_y = nn.BatchNorm1d(self.num_expert_sqrt, affine=False)

        # routed experts
        self.up_embed = nn.Embedding(self.num_experts, self.hidden_size)
        self.down_embed = nn.Embedding(self.num_experts, self.hidden_size)

    def act_fn(self, x: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.silu(x)

    def route(self, hidden_states: torch.Tensor, return_scores: bool = False):
        """Router only: (gates, indices[, scores]) for ``[tokens, hidden]`` input."""
        nx, ny = self.router_norm_x, self.router_norm_y
        if nx.momentum is None or ny.momentum is None:
            raise NotImplementedError("cumulative-average BatchNorm (momentum=None) is not covered")
        return hip_omni_router_fwd_func(
            hidden_states, self.router_gate_x.weight, self.router_gate_y.weight,
            nx.running_mean, nx.running_var, nx.num_batches_tracked,
            ny.running_mean, ny.running_var, ny.num_batches_tracked,
            self.top_k, training=self.training, momentum=nx.momentum, eps=nx.eps, return_scores=return_scores,
        )

    # Router + experts and the gate/up projection only share their input, so they are enqueued
    # on two HIP streams (both at the default priority) and meet again at the down projection,
    # whose epilogue adds the expert output.  Set to False to keep everything on one stream.
    overlap_branches = True

    def _side_stream(self, device) -> "torch.cuda.Stream":
        s = self.__dict__.get("_omni_side_stream")
        if s is None or s.device != device:
            s = torch.cuda.Stream(device=device)
            self.__dict__["_omni_side_stream"] = s
        return s

    def forward(self, hidden_states: torch.Tensor, **kwargs) -> torch.Tensor:
        bsz, seq_len, _ = hidden_states.shape
        with torch.no_grad():
            x = hidden_states.view(-1, self.hidden_size)
            if self.overlap_branches and x.is_cuda:
                main = torch.cuda.current_stream(x.device)
                side = self._side_stream(x.device)
                side.wait_stream(main)                       # x (and the weights) are ready
                with torch.cuda.stream(side):
                    routing_weights, indices = self.route(x)
                    experts_states = hip_omni_expert_func(x, self.up_embed.weight, self.down_embed.weight,
                                                          routing_weights, indices)
                h = hip_swiglu_linear_func(x, self.gate_proj.weight, self.up_proj.weight)
                main.wait_stream(side)
                experts_states.record_stream(main)           # allocated on the side stream, read on this one
                out = hip_linear_func(h, self.down_proj.weight, experts_states)
            else:
                routing_weights, indices = self.route(x)
                experts_states = hip_omni_expert_func(x, self.up_embed.weight, self.down_embed.weight, routing_weights, indices)
                # mlp + experts: the add is the down projection's epilogue
                out = hip_omni_mlp_func(x, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight,
                                        residual=experts_states)
        return out.view(bsz, seq_len, -1)
