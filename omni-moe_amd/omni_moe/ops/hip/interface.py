"""Operator API of the OmniMoE forward path on MI355X.

Same call signatures, shapes, dtypes and return arity as the reference's
``omni_moe/ops/triton/interface.py`` (router :32-51, expert :54-72, mlp :7-29); the
work is done by hand-written gfx950 kernels behind the C ABI in
``include/omni_moe_hip.h``.  Like the reference's operators they are differentiable: when
autograd is recording and an input requires grad, the router, expert and MLP operators go
through ``torch.autograd.Function`` wrappers (``OmniRouterFunc``, ``OmniExpertFunc``,
``OmniSwiGLUFunc``, ``OmniLinearFunc``) whose backward passes are HIP kernels too (GEMM
gradients are library matmuls, as in the reference).  Otherwise no graph is built.
"""
from __future__ import annotations

from typing import NamedTuple, Optional, Tuple

import torch

from . import _lib


def _c(t: torch.Tensor) -> torch.Tensor:
    # the reference makes every tensor argument contiguous (utils.py:47-65)
    return t if t.is_contiguous() else t.contiguous()


def hip_omni_router_func(
    router_logits_x: torch.Tensor,
    router_logits_y: torch.Tensor,
    num_expert_sqrt: int,
    num_experts_per_token: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Cartesian-product top-k: (scores [T,k] in the input dtype, indices [T,k] int32).

    Mirrors ``triton_omni_router_func`` (reference interface.py:32-51) and the input
    contract of ``assert_omni_router_fwd_inputs`` (utils.py:81-104).
    """
    assert router_logits_x.dim() == 2, "router_logits_x must be a 2D tensor of shape (num_tokens, num_expert_sqrt)"
    assert router_logits_y.dim() == 2, "router_logits_y must be a 2D tensor of shape (num_tokens, num_expert_sqrt)"
    assert router_logits_x.size(0) == router_logits_y.size(0), (
        "router_logits_x and router_logits_y must have the same first dimension")
    r, k = int(num_expert_sqrt), int(num_experts_per_token)
    assert 0 <= k <= r * r, f"num_experts_per_token should be in [0, {r * r}], but got {k}"
    assert k <= 128, "num_experts_per_token should be less than or equal to 128"
    assert k % 2 == 0, "num_experts_per_token should be a multiple of 2"
    if router_logits_x.size(1) != r or router_logits_y.size(1) != r:
        raise ValueError("router logits must have num_expert_sqrt columns")
    if router_logits_x.dtype != router_logits_y.dtype or router_logits_x.dtype not in _lib.DTYPE_CODE:
        raise TypeError("router logits must share a dtype in {bfloat16, float16, float32}")
    _lib.require_gpu(router_logits_x, router_logits_y)
    if _needs_grad(router_logits_x, router_logits_y):
        return OmniRouterFunc.apply(router_logits_x, router_logits_y, r, k)
    return _router_select(router_logits_x, router_logits_y, r, k)


def _needs_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _router_select(lx: torch.Tensor, ly: torch.Tensor, r: int, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    lx, ly = _c(lx.detach()), _c(ly.detach())
    dev, T = lx.device, lx.size(0)
    scores = torch.empty((T, k), device=dev, dtype=lx.dtype)
    indices = torch.empty((T, k), device=dev, dtype=torch.int32)
    with torch.cuda.device(dev):
        code = _lib.load().omni_router_select(
            _lib.ptr(lx), _lib.ptr(ly), _lib.ptr(scores), _lib.ptr(indices), T, r, k,
            _lib.DTYPE_CODE[lx.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_router_select")
    return scores, indices


def hip_omni_router_bwd_func(dscores: torch.Tensor, indices: torch.Tensor, num_expert_sqrt: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gradient of the selected scores w.r.t. the two half-logit tensors, each [T, r] in dscores' dtype
    (``_omni_router_backward``, reference omni_router.py:235-274)."""
    if dscores.dim() != 2 or dscores.shape != indices.shape or indices.dtype != torch.int32:
        raise ValueError("dscores and int32 indices must both be (num_tokens, num_experts_per_token)")
    if dscores.dtype not in _lib.DTYPE_CODE:
        raise TypeError("dscores must be bfloat16, float16 or float32")
    dev = _lib.require_gpu(dscores, indices)
    dscores, indices = _c(dscores), _c(indices)
    T, k = dscores.shape
    r = int(num_expert_sqrt)
    dlx = torch.empty((T, r), device=dev, dtype=dscores.dtype)
    dly = torch.empty((T, r), device=dev, dtype=dscores.dtype)
    with torch.cuda.device(dev):
        code = _lib.load().omni_router_bwd(_lib.ptr(dscores), _lib.ptr(indices), _lib.ptr(dlx), _lib.ptr(dly), T, r, k,
                                           _lib.DTYPE_CODE[dscores.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_router_bwd")
    return dlx, dly


class OmniRouterFunc(torch.autograd.Function):
    """Differentiable Cartesian top-k (mirrors ``OmniRouterFunc``, reference omni_router.py:277-307)."""

    @staticmethod
    def forward(ctx, router_logits_x, router_logits_y, num_expert_sqrt, num_experts_per_token):
        scores, indices = _router_select(router_logits_x, router_logits_y, num_expert_sqrt, num_experts_per_token)
        ctx.save_for_backward(indices)
        ctx.num_expert_sqrt = num_expert_sqrt
        ctx.mark_non_differentiable(indices)
        return scores, indices

    @staticmethod
    def backward(ctx, dscores, _dindices):
        (indices,) = ctx.saved_tensors
        dlx, dly = hip_omni_router_bwd_func(dscores, indices, ctx.num_expert_sqrt)
        return dlx, dly, None, None


class Schedule(NamedTuple):
    """Expert-centric layout of the (token, expert) pairs (dense form of the reference's
    ``SchedulingInfo`` tail fields, omni_scheduler.py:5-43)."""
    offsets: torch.Tensor            # [N+1] int32
    sorted_pair_ids: torch.Tensor    # [T*k] int32
    sorted_token_ids: torch.Tensor   # [T*k] int32


def hip_omni_schedule_func(indices: torch.Tensor, num_experts: int) -> Schedule:
    """Counting sort of the pairs by expert id; no device-to-host traffic.

    Stands in for ``get_scheduling_info(G, Indices, num_experts, group_size)``
    (reference omni_scheduler.py:48-101, tail part).
    """
    if indices.dim() != 2 or indices.dtype != torch.int32:
        raise TypeError("indices must be a 2D int32 tensor (num_tokens, num_experts_per_token)")
    dev = _lib.require_gpu(indices)
    idx = _c(indices)
    T, k = idx.shape
    N = int(num_experts)
    lib = _lib.load()
    offsets = torch.empty(N + 1, device=dev, dtype=torch.int32)
    pair_ids = torch.empty(T * k, device=dev, dtype=torch.int32)
    token_ids = torch.empty(T * k, device=dev, dtype=torch.int32)
    ws = torch.empty(max(lib.omni_schedule_workspace_bytes(T, k, N), 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        code = lib.omni_schedule(_lib.ptr(idx), _lib.ptr(offsets), _lib.ptr(pair_ids), _lib.ptr(token_ids),
                                 T, k, N, _lib.ptr(ws), _lib.stream_ptr())
    _lib.check(code, "omni_schedule")
    return Schedule(offsets, pair_ids, token_ids)


_ALGOS = {"auto": _lib.ALGO_AUTO, "gather": _lib.ALGO_GATHER, "segment": _lib.ALGO_SEGMENT, "split": _lib.ALGO_SPLIT, "dense": _lib.ALGO_DENSE}


def hip_omni_expert_func(
    x: torch.Tensor,
    up_weight: torch.Tensor,
    down_weight: torch.Tensor,
    routing_weights: torch.Tensor,
    indices: torch.Tensor,
    algo: str = "auto",
) -> torch.Tensor:
    """y[t] = sum_j silu(<x[t], up[idx_tj]>) * g_tj * down[idx_tj];  y has x's shape and dtype.

    Mirrors ``triton_omni_expert_func`` (reference interface.py:54-72).
    """
    if x.dim() != 2 or up_weight.dim() != 2 or down_weight.dim() != 2:
        raise ValueError("x, up_weight and down_weight must be 2D")
    if routing_weights.shape != indices.shape or routing_weights.dim() != 2 or routing_weights.size(0) != x.size(0):
        raise ValueError("routing_weights and indices must both be (num_tokens, num_experts_per_token)")
    if up_weight.shape != down_weight.shape or up_weight.size(1) != x.size(1):
        raise ValueError("up_weight and down_weight must both be (num_experts, hidden_size)")
    if x.dtype not in _lib.DTYPE_CODE or any(t.dtype != x.dtype for t in (up_weight, down_weight, routing_weights)):
        raise TypeError("x, up_weight, down_weight, routing_weights must share a dtype in {bfloat16, float16, float32}")
    if indices.dtype != torch.int32:
        indices = indices.to(torch.int32)
    _lib.require_gpu(x, up_weight, down_weight, routing_weights, indices)
    if _needs_grad(x, up_weight, down_weight, routing_weights):
        if algo not in ("auto", "gather"):
            raise ValueError("the differentiable expert op uses the default algorithm")
        return OmniExpertFunc.apply(x, up_weight, down_weight, routing_weights, indices)
    return _expert_forward(x, up_weight, down_weight, routing_weights, indices, algo)


def _expert_forward(x, up_weight, down_weight, routing_weights, indices, algo="auto"):
    x, up_weight, down_weight, routing_weights, indices = (
        _c(t.detach()) for t in (x, up_weight, down_weight, routing_weights, indices))
    dev = x.device
    T, H = x.shape
    N, k = up_weight.size(0), indices.size(1)
    lib = _lib.load()
    dt, al = _lib.DTYPE_CODE[x.dtype], _ALGOS[algo]
    y = torch.empty_like(x)
    nbytes = lib.omni_expert_workspace_bytes(T, H, N, k, dt, al)
    ws = torch.empty(nbytes, device=dev, dtype=torch.uint8) if nbytes else None
    with torch.cuda.device(dev):
        code = lib.omni_expert_fwd(_lib.ptr(x), _lib.ptr(up_weight), _lib.ptr(down_weight), _lib.ptr(routing_weights),
                                   _lib.ptr(indices), _lib.ptr(y), T, H, N, k, dt, al, _lib.ptr(ws), _lib.stream_ptr())
    _lib.check(code, "omni_expert_fwd")
    return y


def hip_omni_expert_bwd_func(dy, x, up_weight, down_weight, routing_weights, indices):
    """Gradients of the expert op: (dx [T,H], dup_weight [N,H], ddown_weight [N,H], drouting_weights [T,k]),
    each in the dtype of its primal (``omni_expert_backward``, reference omni_expert.py:1067-1277)."""
    if dy.shape != x.shape or dy.dtype != x.dtype:
        raise ValueError("dy must match x in shape and dtype")
    dev = _lib.require_gpu(dy, x, up_weight, down_weight, routing_weights, indices)
    dy, x, up_weight, down_weight, routing_weights, indices = map(_c, (dy, x, up_weight, down_weight, routing_weights, indices))
    T, H = x.shape
    N, k = up_weight.size(0), indices.size(1)
    lib = _lib.load()
    dt = _lib.DTYPE_CODE[x.dtype]
    dx, dup, ddown, dg = torch.empty_like(x), torch.empty_like(up_weight), torch.empty_like(down_weight), torch.empty_like(routing_weights)
    ws = torch.empty(max(lib.omni_expert_bwd_workspace_bytes(T, H, N, k, dt), 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        code = lib.omni_expert_bwd(_lib.ptr(dy), _lib.ptr(x), _lib.ptr(up_weight), _lib.ptr(down_weight), _lib.ptr(routing_weights),
                                   _lib.ptr(indices), _lib.ptr(dx), _lib.ptr(dup), _lib.ptr(ddown), _lib.ptr(dg), T, H, N, k, dt,
                                   _lib.ptr(ws), _lib.stream_ptr())
    _lib.check(code, "omni_expert_bwd")
    return dx, dup, ddown, dg


class OmniExpertFunc(torch.autograd.Function):
    """Differentiable fused expert op (mirrors ``OmniExpertFunc``, reference omni_expert.py:1280-1360).
    Only the inputs are saved: the backward recomputes the pair scores."""

    @staticmethod
    def forward(ctx, x, up_weight, down_weight, routing_weights, indices):
        y = _expert_forward(x, up_weight, down_weight, routing_weights, indices)
        ctx.save_for_backward(x, up_weight, down_weight, routing_weights, indices)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, up_weight, down_weight, routing_weights, indices = ctx.saved_tensors
        dx, dup, ddown, dg = hip_omni_expert_bwd_func(dy, x, up_weight, down_weight, routing_weights, indices)
        return dx, dup, ddown, dg, None


def hip_omni_mlp_func(
    x: torch.Tensor,
    gate_weight: torch.Tensor,
    up_weight: torch.Tensor,
    down_weight: torch.Tensor,
    residual: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """(silu(x gate^T) * (x up^T)) down^T, optionally + residual;  y has x's shape and dtype.

    Mirrors ``triton_omni_mlp_func`` (reference interface.py:7-29).  ``residual`` has no
    counterpart there: the layer uses it to fold its final ``mlp + experts`` add
    (omni_moe.py:102) into the down projection's epilogue.
    """
    if x.dim() != 2 or gate_weight.dim() != 2 or up_weight.dim() != 2 or down_weight.dim() != 2:
        raise ValueError("x and the three weights must be 2D")
    T, H = x.shape
    I = gate_weight.size(0)
    if gate_weight.shape != (I, H) or up_weight.shape != (I, H) or down_weight.shape != (H, I):
        raise ValueError("expected gate/up weights (intermediate, hidden) and down weight (hidden, intermediate)")
    if x.dtype not in _lib.DTYPE_CODE or any(t.dtype != x.dtype for t in (gate_weight, up_weight, down_weight)):
        raise TypeError("x and the weights must share a dtype in {bfloat16, float16, float32}")
    tensors = [x, gate_weight, up_weight, down_weight]
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("residual must match x in shape and dtype")
        tensors.append(residual)
    dev = _lib.require_gpu(*tensors)
    if _needs_grad(*tensors):
        # the reference's composition (interface.py:23-29): three matmuls around the SwiGLU function.  Where the fused
        # kernel can keep gate and up for the backward pass, the first two matmuls and the SwiGLU are one launch.
        if _swiglu_linear_save_covers(x, gate_weight):
            h = OmniSwiGLULinearFunc.apply(x, gate_weight, up_weight)
        else:
            gate = OmniLinearFunc.apply(x, gate_weight)
            up = OmniLinearFunc.apply(x, up_weight)
            h = OmniSwiGLUFunc.apply(gate, up)
        y = OmniLinearFunc.apply(h, down_weight)
        return y if residual is None else y + residual
    x, gate_weight, up_weight, down_weight = (_c(t.detach()) for t in (x, gate_weight, up_weight, down_weight))
    residual = _c(residual.detach()) if residual is not None else None
    lib = _lib.load()
    dt = _lib.DTYPE_CODE[x.dtype]
    y = torch.empty_like(x)
    ws = torch.empty(max(lib.omni_mlp_workspace_bytes(T, H, I, dt), 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        code = lib.omni_mlp_fwd(_lib.ptr(x), _lib.ptr(gate_weight), _lib.ptr(up_weight), _lib.ptr(down_weight),
                                _lib.ptr(residual), _lib.ptr(y), T, H, I, dt, _lib.ptr(ws), _lib.stream_ptr())
    _lib.check(code, "omni_mlp_fwd")
    return y


def hip_linear_func(x: torch.Tensor, weight: torch.Tensor, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x @ weight.T (+ residual) for a bias-free ``nn.Linear`` (reference omni_moe.py:70-71, interface.py:23-29)."""
    if x.dim() != 2 or weight.dim() != 2 or weight.size(1) != x.size(1):
        raise ValueError("expected x (tokens, in) and weight (out, in)")
    if x.dtype not in _lib.DTYPE_CODE or weight.dtype != x.dtype:
        raise TypeError("x and weight must share a dtype in {bfloat16, float16, float32}")
    if residual is not None and (residual.shape != (x.size(0), weight.size(0)) or residual.dtype != x.dtype):
        raise ValueError("residual must be (tokens, out) in x's dtype")
    _lib.require_gpu(x, weight)
    if _needs_grad(x, weight, residual):
        y = OmniLinearFunc.apply(x, weight)
        return y if residual is None else y + residual
    return _linear_forward(x, weight, residual)


def _linear_forward(x, weight, residual=None):
    x, weight = _c(x.detach()), _c(weight.detach())
    residual = _c(residual.detach()) if residual is not None else None
    dev = x.device
    y = torch.empty((x.size(0), weight.size(0)), device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        code = _lib.load().omni_linear_fwd(_lib.ptr(x), _lib.ptr(weight), _lib.ptr(residual), _lib.ptr(y), x.size(0), x.size(1),
                                           weight.size(0), _lib.DTYPE_CODE[x.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_linear_fwd")
    return y


class OmniLinearFunc(torch.autograd.Function):
    """y = x W^T with the forward on the gfx950 GEMM; the two gradient GEMMs are library matmuls, as the
    reference's ``torch.matmul`` calls get from autograd (interface.py:23-29)."""

    @staticmethod
    def forward(ctx, x, weight):
        ctx.save_for_backward(x, weight)
        return _linear_forward(x, weight)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dx = dy.matmul(weight) if ctx.needs_input_grad[0] else None
        dw = dy.t().matmul(x) if ctx.needs_input_grad[1] else None
        return dx, dw


def hip_swiglu_func(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up element-wise, fp32 inside, one rounding (``TritonSwiGLUFunc``, reference omni_mlp.py:359-371)."""
    assert gate.shape == up.shape, "gate and up must have the same shape"       # the reference asserts (utils.py:68-78)
    if gate.dtype != up.dtype or gate.dtype not in _lib.DTYPE_CODE:
        raise ValueError("gate and up must share one dtype (bfloat16, float16 or float32)")
    _lib.require_gpu(gate, up)
    if _needs_grad(gate, up):
        return OmniSwiGLUFunc.apply(gate, up)
    return _swiglu_forward(gate, up)


def _swiglu_forward(gate, up):
    gate, up = _c(gate.detach()), _c(up.detach())
    out = torch.empty_like(gate)
    with torch.cuda.device(gate.device):
        code = _lib.load().omni_swiglu_fwd(_lib.ptr(gate), _lib.ptr(up), _lib.ptr(out), gate.numel(),
                                           _lib.DTYPE_CODE[gate.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_swiglu_fwd")
    return out


def hip_swiglu_bwd_func(dout, gate, up):
    """(dgate, dup) of ``hip_swiglu_func`` (reference omni_mlp.py:306-356)."""
    assert dout.shape == gate.shape == up.shape, "dout, gate and up must have the same shape"
    if len({dout.dtype, gate.dtype, up.dtype}) != 1:
        raise ValueError("dout, gate and up must share one dtype")
    _lib.require_gpu(dout, gate, up)
    dout, gate, up = _c(dout), _c(gate), _c(up)
    dgate, dup = torch.empty_like(gate), torch.empty_like(up)
    with torch.cuda.device(gate.device):
        code = _lib.load().omni_swiglu_bwd(_lib.ptr(dout), _lib.ptr(gate), _lib.ptr(up), _lib.ptr(dgate), _lib.ptr(dup),
                                           gate.numel(), _lib.DTYPE_CODE[gate.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_swiglu_bwd")
    return dgate, dup


def _swiglu_linear_save_covers(x, gate_weight) -> bool:
    """Shapes the saving form of the fused gate/up GEMM takes (omni_swiglu_linear_save_fwd)."""
    return x.dtype in (torch.bfloat16, torch.float16) and gate_weight.size(0) % 8 == 0 and x.size(1) % 64 == 0


class OmniSwiGLULinearFunc(torch.autograd.Function):
    """h = silu(x Wg^T) * (x Wu^T) as ONE GEMM launch that also keeps the rounded gate and up projections, which is all
    the backward pass needs: the first three steps of ``triton_omni_mlp_func`` (reference interface.py:23-27, with
    ``TritonSwiGLUFunc`` saving gate and up, omni_mlp.py:359-371)."""

    @staticmethod
    def forward(ctx, x, gate_weight, up_weight):
        xd, wg, wu = _c(x.detach()), _c(gate_weight.detach()), _c(up_weight.detach())
        T, I = xd.size(0), wg.size(0)
        h = torch.empty(T, I, device=xd.device, dtype=xd.dtype)
        gate, up = torch.empty_like(h), torch.empty_like(h)
        with torch.cuda.device(xd.device):
            code = _lib.load().omni_swiglu_linear_save_fwd(_lib.ptr(xd), _lib.ptr(wg), _lib.ptr(wu), _lib.ptr(h), _lib.ptr(gate), _lib.ptr(up),
                                                           T, xd.size(1), I, _lib.DTYPE_CODE[xd.dtype], _lib.stream_ptr())
        _lib.check(code, "omni_swiglu_linear_save_fwd")
        ctx.save_for_backward(xd, wg, wu, gate, up)
        return h

    @staticmethod
    def backward(ctx, dh):
        x, wg, wu, gate, up = ctx.saved_tensors
        dgate, dup = hip_swiglu_bwd_func(dh, gate, up)
        dx = dw_g = dw_u = None
        if ctx.needs_input_grad[0]:
            dx = torch.addmm(dgate.matmul(wg), dup, wu)
        if ctx.needs_input_grad[1]:
            dw_g = dgate.t().matmul(x)
        if ctx.needs_input_grad[2]:
            dw_u = dup.t().matmul(x)
        return dx, dw_g, dw_u


class OmniSwiGLUFunc(torch.autograd.Function):
    """Differentiable element-wise SwiGLU (mirrors ``TritonSwiGLUFunc``, reference omni_mlp.py:359-371)."""

    @staticmethod
    def forward(ctx, gate, up):
        ctx.save_for_backward(gate, up)
        return _swiglu_forward(gate, up)

    @staticmethod
    def backward(ctx, dout):
        gate, up = ctx.saved_tensors
        return hip_swiglu_bwd_func(dout, gate, up)


def hip_swiglu_linear_func(x: torch.Tensor, gate_weight: torch.Tensor, up_weight: torch.Tensor, shared: bool = False) -> torch.Tensor:
    """silu(x gate^T) * (x up^T): the first half of the MLP op as one GEMM with a fused epilogue.  ``shared=True`` says that
    other kernels run beside it (another stream): the launch then never takes the form that holds every CU."""
    if x.dim() != 2 or gate_weight.shape != up_weight.shape or gate_weight.dim() != 2 or gate_weight.size(1) != x.size(1):
        raise ValueError("expected x (tokens, hidden) and gate/up weights (intermediate, hidden)")
    if x.dtype not in _lib.DTYPE_CODE or gate_weight.dtype != x.dtype or up_weight.dtype != x.dtype:
        raise TypeError("x and the weights must share a dtype in {bfloat16, float16, float32}")
    dev = _lib.require_gpu(x, gate_weight, up_weight)
    x, gate_weight, up_weight = map(_c, (x, gate_weight, up_weight))
    h = torch.empty((x.size(0), gate_weight.size(0)), device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        fn = _lib.load().omni_swiglu_linear_fwd_shared if shared else _lib.load().omni_swiglu_linear_fwd
        code = fn(_lib.ptr(x), _lib.ptr(gate_weight), _lib.ptr(up_weight), _lib.ptr(h), x.size(0), x.size(1), gate_weight.size(0),
                  _lib.DTYPE_CODE[x.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_swiglu_linear_fwd")
    return h


def hip_add_inplace_func(y: torch.Tensor, addend: torch.Tensor) -> torch.Tensor:
    """y += addend, rounded once (the layer's final ``mlp + experts``, reference omni_moe.py:102)."""
    if y.shape != addend.shape or y.dtype != addend.dtype or y.dtype not in _lib.DTYPE_CODE:
        raise ValueError("y and addend must match in shape and dtype (bfloat16, float16 or float32)")
    if not (y.is_contiguous() and addend.is_contiguous()):
        raise ValueError("y and addend must be contiguous")
    dev = _lib.require_gpu(y, addend)
    with torch.cuda.device(dev):
        code = _lib.load().omni_add_inplace(_lib.ptr(y), _lib.ptr(addend), y.numel(), _lib.DTYPE_CODE[y.dtype], _lib.stream_ptr())
    _lib.check(code, "omni_add_inplace")
    return y


def hip_omni_router_fwd_func(
    x: torch.Tensor,
    weight_x: torch.Tensor,
    weight_y: torch.Tensor,
    running_mean_x: torch.Tensor,
    running_var_x: torch.Tensor,
    num_batches_tracked_x: Optional[torch.Tensor],
    running_mean_y: torch.Tensor,
    running_var_y: torch.Tensor,
    num_batches_tracked_y: Optional[torch.Tensor],
    num_experts_per_token: int,
    training: bool,
    momentum: float = 0.1,
    eps: float = 1e-5,
    return_scores: bool = False,
):
    """Router of the layer in one call: projection -> BatchNorm1d(affine=False) ->
    log_softmax -> Cartesian top-k -> exp  (reference omni_moe/modules/omni_moe.py:70-86).

    Returns (gates [T,k] in x's dtype, indices [T,k] int32[, scores]).  In training mode the
    running buffers are updated in place, as nn.BatchNorm1d does.
    """
    if x.dim() != 2 or weight_x.shape != weight_y.shape or weight_x.dim() != 2 or weight_x.size(1) != x.size(1):
        raise ValueError("expected x (tokens, hidden) and two router weights (num_expert_sqrt, hidden)")
    if x.dtype not in _lib.DTYPE_CODE or weight_x.dtype != x.dtype or weight_y.dtype != x.dtype:
        raise TypeError("x and the router weights must share a dtype in {bfloat16, float16, float32}")
    stats = (running_mean_x, running_var_x, running_mean_y, running_var_y)
    r, k = weight_x.size(0), int(num_experts_per_token)
    if any(t.dtype != running_mean_x.dtype or t.shape != (r,) or not t.is_contiguous() for t in stats):
        raise ValueError("running statistics must be contiguous (num_expert_sqrt,) tensors of one dtype")
    if running_mean_x.dtype not in _lib.DTYPE_CODE:
        raise TypeError("running statistics must be bfloat16, float16 or float32")
    assert 0 <= k <= r * r, f"num_experts_per_token should be in [0, {r * r}], but got {k}"
    assert k <= 128, "num_experts_per_token should be less than or equal to 128"
    assert k % 2 == 0, "num_experts_per_token should be a multiple of 2"
    for nbt in (num_batches_tracked_x, num_batches_tracked_y):
        if nbt is not None and (nbt.dtype != torch.int64 or nbt.numel() != 1):
            raise TypeError("num_batches_tracked must be an int64 scalar tensor")
    _check_batch_norm_call(x.size(0), r, training, momentum, num_batches_tracked_x, num_batches_tracked_y)
    momentum = -1.0 if momentum is None else momentum
    _lib.require_gpu(x, weight_x, weight_y, *stats)
    if _needs_grad(x, weight_x, weight_y):
        if return_scores:
            raise ValueError("the differentiable router stage returns gates and indices only")
        return OmniRouterStageFunc.apply(x, weight_x, weight_y, running_mean_x, running_var_x, num_batches_tracked_x,
                                         running_mean_y, running_var_y, num_batches_tracked_y, k, bool(training),
                                         float(momentum), float(eps))
    out = _router_stage_forward(x, weight_x, weight_y, running_mean_x, running_var_x, num_batches_tracked_x,
                                running_mean_y, running_var_y, num_batches_tracked_y, k, training, momentum, eps, return_scores)
    return out[:3] if return_scores else out[:2]


def _check_batch_norm_call(num_tokens, r, training, momentum, nbt_x, nbt_y):
    """What nn.BatchNorm1d checks itself (reference omni_moe.py:53-54,70-71)."""
    if training and num_tokens == 1:
        raise ValueError(f"Expected more than 1 value per channel when training, got input size torch.Size([1, {r}])")
    if training and momentum is None and (nbt_x is None or nbt_y is None):
        raise ValueError("momentum=None (cumulative moving average) needs num_batches_tracked")


def _router_stage_forward(x, weight_x, weight_y, running_mean_x, running_var_x, num_batches_tracked_x,
                          running_mean_y, running_var_y, num_batches_tracked_y, k, training, momentum, eps, return_scores=False):
    """(gates, indices, scores or None, workspace): the workspace still holds z and the BatchNorm statistics."""
    x, weight_x, weight_y = (_c(t.detach()) for t in (x, weight_x, weight_y))
    dev, r = x.device, weight_x.size(0)
    T, H = x.shape
    lib = _lib.load()
    dt = _lib.DTYPE_CODE[x.dtype]
    gates = torch.empty((T, k), device=dev, dtype=x.dtype)
    indices = torch.empty((T, k), device=dev, dtype=torch.int32)
    scores = torch.empty((T, k), device=dev, dtype=x.dtype) if return_scores else None
    ws = torch.empty(max(lib.omni_router_workspace_bytes(T, r, dt), 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        code = lib.omni_router_fwd(
            _lib.ptr(x), _lib.ptr(weight_x), _lib.ptr(weight_y),
            _lib.ptr(running_mean_x), _lib.ptr(running_var_x), _lib.ptr(num_batches_tracked_x),
            _lib.ptr(running_mean_y), _lib.ptr(running_var_y), _lib.ptr(num_batches_tracked_y),
            1 if training else 0, float(momentum), float(eps), _lib.ptr(gates), _lib.ptr(indices), _lib.ptr(scores),
            T, H, r, k, dt, _lib.DTYPE_CODE[running_mean_x.dtype], _lib.ptr(ws), _lib.stream_ptr())
    _lib.check(code, "omni_router_fwd")
    return gates, indices, scores, ws


def hip_omni_router_stage_bwd_func(dgates, gates, indices, workspace, num_tokens, num_expert_sqrt, training):
    """d(z) [T, 2r] of the router stage from d(gates), using z and the statistics that ``omni_router_fwd`` left in
    ``workspace`` (exp, router op, log_softmax and BatchNorm1d of reference omni_moe.py:70-86 in reverse)."""
    lib = _lib.load()
    dev = _lib.require_gpu(dgates, gates, indices, workspace)
    T, r, k = int(num_tokens), int(num_expert_sqrt), gates.size(1)
    dt = _lib.DTYPE_CODE[gates.dtype]
    dgates = _c(dgates)
    off = lib.omni_router_workspace_stats_offset(T, r, dt)
    dz = torch.empty((T, 2 * r), device=dev, dtype=gates.dtype)
    ws = torch.empty(max(lib.omni_router_norm_bwd_workspace_bytes(T, r), 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        code = lib.omni_router_norm_bwd(_lib.ptr(dgates), _lib.ptr(gates), _lib.ptr(indices), workspace.data_ptr(),
                                        workspace.data_ptr() + off, _lib.ptr(dz), T, r, k, dt, 1 if training else 0,
                                        _lib.ptr(ws), _lib.stream_ptr())
    _lib.check(code, "omni_router_norm_bwd")
    return dz


class OmniRouterStageFunc(torch.autograd.Function):
    """The layer's router (projection, BatchNorm1d, log_softmax, router op, exp; reference omni_moe.py:70-86) as one
    differentiable node: the forward is ``omni_router_fwd``, the backward one HIP pass from d(gates) to d(z) and the two
    library GEMMs for d(weights) and d(x)."""

    @staticmethod
    def forward(ctx, x, weight_x, weight_y, rmx, rvx, nbtx, rmy, rvy, nbty, k, training, momentum, eps):
        gates, indices, _, ws = _router_stage_forward(x, weight_x, weight_y, rmx, rvx, nbtx, rmy, rvy, nbty, k, training,
                                                      momentum, eps)
        ctx.save_for_backward(x, weight_x, weight_y, gates, indices, ws)
        ctx.training = training
        ctx.mark_non_differentiable(indices)
        return gates, indices

    @staticmethod
    def backward(ctx, dgates, _dindices):
        x, weight_x, weight_y, gates, indices, ws = ctx.saved_tensors
        r = weight_x.size(0)
        dz = hip_omni_router_stage_bwd_func(dgates, gates, indices, ws, x.size(0), r, ctx.training)
        dw = dz.t().matmul(x) if (ctx.needs_input_grad[1] or ctx.needs_input_grad[2]) else None
        dx = dz.matmul(torch.cat([weight_x, weight_y])) if ctx.needs_input_grad[0] else None
        return (dx, dw[:r] if dw is not None else None, dw[r:] if dw is not None else None) + (None,) * 10


def hip_omni_moe_fwd_func(
    x: torch.Tensor,
    gate_weight: torch.Tensor, up_weight: torch.Tensor, down_weight: torch.Tensor,
    router_weight_x: torch.Tensor, router_weight_y: torch.Tensor,
    running_mean_x: torch.Tensor, running_var_x: torch.Tensor, num_batches_tracked_x: Optional[torch.Tensor],
    running_mean_y: torch.Tensor, running_var_y: torch.Tensor, num_batches_tracked_y: Optional[torch.Tensor],
    up_embed: torch.Tensor, down_embed: torch.Tensor,
    num_experts_per_token: int, training: bool, momentum: float = 0.1, eps: float = 1e-5,
    side_stream: Optional["torch.cuda.Stream"] = None,
    fork_event: Optional["torch.cuda.Event"] = None, join_event: Optional["torch.cuda.Event"] = None,
    expert_algo: str = "auto",
) -> torch.Tensor:
    """The whole layer forward (reference omni_moe.py:60-106) for ``x`` of shape (tokens, hidden) in one
    library call.  With ``side_stream`` (and two events) the router + expert branch is enqueued next
    to the MLP branch; the current stream waits for it before the final add.  ``expert_algo`` names the
    expert algorithm ("auto" decides from the sizes alone)."""
    T, H = x.shape
    I, N, r, k = gate_weight.size(0), up_embed.size(0), router_weight_x.size(0), int(num_experts_per_token)
    weights = (gate_weight, up_weight, down_weight, router_weight_x, router_weight_y, up_embed, down_embed)
    if x.dim() != 2 or x.dtype not in _lib.DTYPE_CODE or any(t.dtype != x.dtype for t in weights):
        raise TypeError("x and the weights must share a dtype in {bfloat16, float16, float32}")
    if (gate_weight.shape != (I, H) or up_weight.shape != (I, H) or down_weight.shape != (H, I) or router_weight_y.shape != (r, H)
            or router_weight_x.shape != (r, H) or up_embed.shape != (N, H) or down_embed.shape != (N, H)):
        raise ValueError("weight shapes do not fit (tokens, hidden) input")
    stats = (running_mean_x, running_var_x, running_mean_y, running_var_y)
    if any(t.dtype != running_mean_x.dtype or t.shape != (r,) or not t.is_contiguous() for t in stats) or running_mean_x.dtype not in _lib.DTYPE_CODE:
        raise ValueError("running statistics must be contiguous (num_expert_sqrt,) tensors of one floating dtype")
    assert 0 <= k <= r * r, f"num_experts_per_token should be in [0, {r * r}], but got {k}"
    assert k <= 128, "num_experts_per_token should be less than or equal to 128"
    assert k % 2 == 0, "num_experts_per_token should be a multiple of 2"
    _check_batch_norm_call(T, r, training, momentum, num_batches_tracked_x, num_batches_tracked_y)
    momentum = -1.0 if momentum is None else momentum
    dev = _lib.require_gpu(x, *weights, *stats)
    x = _c(x)
    # the reference makes every tensor argument of its operators contiguous (utils.py:47-65)
    gate_weight, up_weight, down_weight, router_weight_x, router_weight_y, up_embed, down_embed = (_c(t) for t in weights)
    lib = _lib.load()
    dt = _lib.DTYPE_CODE[x.dtype]
    y = torch.empty_like(x)
    if expert_algo not in _ALGOS:
        raise ValueError(f"expert_algo must be one of {sorted(_ALGOS)}")
    al = _ALGOS[expert_algo]
    ws = torch.empty(max(lib.omni_moe_workspace_bytes_algo(T, H, I, N, r, k, dt, al), 1), device=dev, dtype=torch.uint8)
    side = fork = join = 0
    if side_stream is not None:
        side, fork, join = side_stream.cuda_stream, fork_event.cuda_event, join_event.cuda_event
    with torch.cuda.device(dev):
        code = lib.omni_moe_fwd_algo(
            _lib.ptr(x), _lib.ptr(gate_weight), _lib.ptr(up_weight), _lib.ptr(down_weight), _lib.ptr(router_weight_x),
            _lib.ptr(router_weight_y), _lib.ptr(running_mean_x), _lib.ptr(running_var_x), _lib.ptr(num_batches_tracked_x),
            _lib.ptr(running_mean_y), _lib.ptr(running_var_y), _lib.ptr(num_batches_tracked_y), _lib.ptr(up_embed),
            _lib.ptr(down_embed), _lib.ptr(y), T, H, I, N, r, k, dt, _lib.DTYPE_CODE[running_mean_x.dtype],
            1 if training else 0, float(momentum), float(eps), _lib.ptr(ws), _lib.stream_ptr(), side, fork, join, al)
    _lib.check(code, "omni_moe_fwd_algo")
    # ws is released here: the current stream has been made to wait for the side branch, so every
    # later use of that memory (allocated from this stream's pool) is ordered after both branches
    return y
