"""OmniMoE layer: drop-in for the reference's ``omni_moe.modules.omni_moe`` (forward path).

Same constructor, attribute / ``state_dict`` names and ``forward(hidden_states, **kwargs)``
as the reference's ``OmniMoE`` (omni_moe/modules/omni_moe.py:14-106); the forward is ONE call
into the gfx950 library (``omni_moe_fwd``): router (projection, BatchNorm, log-softmax,
Cartesian top-k, exp) and fused experts on a side stream, the shared SwiGLU MLP on the
caller's stream, joined by the final add (``overlap_branches = False``: everything on the
caller's stream, the add fused into the down projection).

When autograd is recording and the input or a parameter requires grad, ``forward`` instead
composes differentiable operators in the reference's order (omni_moe.py:64-104: the router
stage -- Linear, BatchNorm1d, log_softmax, router op, exp -- as one node, the expert op, the
MLP op, add), so the layer trains; call it under ``torch.no_grad()`` for the fused path.
"""
import math
import threading

import torch
import torch.nn as nn

from omni_moe.ops.hip import hip_omni_expert_func, hip_omni_mlp_func, hip_omni_moe_fwd_func, hip_omni_router_fwd_func


_BRANCH_RESOURCES = {}      # (device index, host thread) -> (side stream, fork event, join event)


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

    def _router_norms(self):
        """The two BatchNorm modules; the library applies one momentum and one eps to both halves."""
        nx, ny = self.router_norm_x, self.router_norm_y
        if nx.momentum != ny.momentum or nx.eps != ny.eps:
            raise ValueError("router_norm_x and router_norm_y must share momentum and eps")
        return nx, ny

    def route(self, hidden_states: torch.Tensor, return_scores: bool = False):
        """Router only: (gates, indices[, scores]) for ``[tokens, hidden]`` input."""
        nx, ny = self._router_norms()
        return hip_omni_router_fwd_func(
            hidden_states, self.router_gate_x.weight, self.router_gate_y.weight,
            nx.running_mean, nx.running_var, nx.num_batches_tracked,
            ny.running_mean, ny.running_var, ny.num_batches_tracked,
            self.top_k, training=self.training, momentum=nx.momentum, eps=nx.eps, return_scores=return_scores,
        )

    # Router + experts and the shared MLP only share their input, so the library enqueues them on
    # two HIP streams (both at the default priority) and joins them at the final add: the expert
    # kernel (cache bandwidth, no LDS) shares CUs with the projections (LDS and MFMA).  Set to False
    # to keep everything on one stream, with the add as the down projection's epilogue.
    overlap_branches = True
    # The fork and join cost about 50 us of host time per call, so below this much work (tokens x hidden x
    # intermediate; 2048 x 1024 x 4096 measured level on an MI355X) the call would be host-bound: one stream then.
    overlap_min_work = 2 ** 33
    # ... and from this much work on, one stream is the faster schedule again: the chip is power-limited under the GEMMs, so
    # overlapped kernels slow each other by about what they would cost alone, and the fork and join are not free
    # (measured, hidden 1024 x intermediate 4096, two streams against one: 4096 tokens 126 against 135 us, 8192 tokens 229
    # against 241, 16384 tokens 425-440 against 415, 65536 tokens 1.66-1.70 against 1.63 ms; benchmark config 5: 3.43 against 3.17 ms).
    overlap_max_work = 2 ** 36
    # Expert algorithm of the fused forward: "auto" decides from the sizes alone (no device-to-host read).  Which one is
    # faster also depends on how many DISTINCT experts the router picks: auto's rule is fitted to ids spread evenly
    # over the tables, and a router that concentrates on few experts moves the crossover between "gather" and "split";
    # the caller who knows the distribution says so here.
    expert_algo = "auto"

    @staticmethod
    def _branch_resources(device):
        """Side stream and the fork / join events for ``device``, one set per device and host thread.  They live in a
        table of this module, not on the layer: a layer stays a plain ``nn.Module`` that ``copy.deepcopy``,
        ``torch.save`` and ``state_dict`` treat as the reference's, and layers that run one after another on a
        stream share the set (an event is recorded and waited for again by every call)."""
        key = (device.index if device.index is not None else torch.cuda.current_device(), threading.get_ident())
        res = _BRANCH_RESOURCES.get(key)
        if res is None:
            with torch.cuda.device(device):
                side = torch.cuda.Stream(device=device)
                fork, join = torch.cuda.Event(), torch.cuda.Event()
                fork.record()                                # events come into being when first recorded
                join.record()
            res = _BRANCH_RESOURCES[key] = (side, fork, join)
        return res

    def _forward_differentiable(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """The reference's composition (omni_moe.py:64-104) over the differentiable operators."""
        bsz, seq_len, _ = hidden_states.shape
        x = hidden_states.reshape(-1, self.hidden_size)
        routing_weights, indices = self.route(x)          # one differentiable node (OmniRouterStageFunc)
        experts_states = hip_omni_expert_func(x, self.up_embed.weight, self.down_embed.weight, routing_weights, indices)
        mlp_states = hip_omni_mlp_func(x, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight)
        return (mlp_states + experts_states).view(bsz, seq_len, -1)

    def forward(self, hidden_states: torch.Tensor, **kwargs) -> torch.Tensor:
        bsz, seq_len, _ = hidden_states.shape
        if torch.is_grad_enabled() and (hidden_states.requires_grad or any(p.requires_grad for p in self.parameters())):
            return self._forward_differentiable(hidden_states)
        nx, ny = self._router_norms()
        with torch.no_grad():
            x = hidden_states.view(-1, self.hidden_size)
            work = x.size(0) * self.hidden_size * self.intermediate_size
            two = self.overlap_branches and x.is_cuda and self.overlap_min_work < work < self.overlap_max_work
            side, fork, join = self._branch_resources(x.device) if two else (None, None, None)
            out = hip_omni_moe_fwd_func(
                x, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight,
                self.router_gate_x.weight, self.router_gate_y.weight,
                nx.running_mean, nx.running_var, nx.num_batches_tracked,
                ny.running_mean, ny.running_var, ny.num_batches_tracked,
                self.up_embed.weight, self.down_embed.weight, self.top_k,
                training=self.training, momentum=nx.momentum, eps=nx.eps,
                side_stream=side, fork_event=fork, join_event=join, expert_algo=self.expert_algo)
        return out.view(bsz, seq_len, -1)
