"""CPU oracle for the OmniMoE forward path.  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only the test-suite, the smoke
check and the CPU-baseline leg of the benchmark may import it.  The shipped
package (``omni_moe``) never imports it and never falls back to it.

It restates, with torch *library* routines on the CPU, the algorithm of the
reference's pure-PyTorch layer ``OmniMoE_Torch.forward``
(reference ``omni_moe/modules/omni_moe.py:139-194``) and of the three in-test
restatements the reference's own benchmarks carry
(``tests/test_router.py:8-22``, ``tests/test_expert.py:8-25``,
``tests/test_mlp.py:8-21``).  The reference ships no golden vectors; every
function below is pinned in ``tests/test_oracle.py`` against an independent
formulation (a torch library routine of the same mathematics, a brute-force
loop on tiny inputs, or an invariant), listed per function:

* ``batch_norm``        <- ``torch.nn.functional.batch_norm`` (train and eval) and
                           ``nn.BatchNorm1d`` buffer updates
* ``log_softmax``       <- ``torch.log_softmax``; invariant logsumexp(out)=0
* ``router_select``     <- brute force over the full r*r outer sum (values equal
                           ``torch.topk`` bit for bit; ids recompute their score;
                           ids equal topk's where scores are distinct; explicit
                           tie cases with the lower-position rule)
* ``schedule``          <- ``torch.bincount`` / ``torch.sort(stable=True)``; loop
* ``expert_forward``    <- per-token python loop; linearity / permutation /
                           duplicate-id invariants
* ``mlp_forward``       <- ``F.silu`` + three matmuls in float64
* ``moe_forward``       <- composition; an ``nn.Module`` built from torch layers
                           following the reference's layer definition

The one behaviour the reference leaves to the library is the order of ties in
``torch.topk``.  The oracle fixes it: per half, equal scores keep the lower key
index first; among candidate sums, equal scores keep the lower candidate
position ``a*k'+b`` first (the rule of the reference kernel's ``argmax``,
``omni_moe/ops/triton/omni_router.py:74-95``).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

BN_EPS = 1e-5        # nn.BatchNorm1d default, reference omni_moe.py:53-54
BN_MOMENTUM = 0.1    # nn.BatchNorm1d default


# --------------------------------------------------------------------------
# router
# --------------------------------------------------------------------------
def _stable_topk_desc(v: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k along the last axis, descending, ties -> lower index first."""
    s, i = torch.sort(v.float(), dim=-1, descending=True, stable=True)
    return s[..., :k].to(v.dtype), i[..., :k]


def router_select(
    lx: torch.Tensor, ly: torch.Tensor, num_expert_sqrt: int, num_experts_per_token: int
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Cartesian-product top-k.

    Follows ``_omni_router_forward`` (reference omni_router.py:167-232): per-half
    top-k' with k' = min(r, k) (:180,186-189), candidate sums formed in the INPUT
    dtype (:66-70; torch twin omni_moe.py:168), k selections by descending score,
    expert id = ix*r + iy (:88), scores in the input dtype and ids int32 (:192-201).
    """
    r, k = num_expert_sqrt, num_experts_per_token
    assert lx.dim() == 2 and ly.dim() == 2 and lx.size(0) == ly.size(0)
    assert 0 <= k <= r * r and k <= 128 and k % 2 == 0   # reference utils.py:81-104
    kp = min(r, k)
    sx, ix = _stable_topk_desc(lx, kp)
    sy, iy = _stable_topk_desc(ly, kp)
    cand = (sx.unsqueeze(-1) + sy.unsqueeze(-2)).reshape(lx.size(0), kp * kp)  # input dtype add
    ids = (ix.unsqueeze(-1) * r + iy.unsqueeze(-2)).reshape(lx.size(0), kp * kp)
    s, pos = torch.sort(cand.float(), dim=-1, descending=True, stable=True)
    pos = pos[:, :k]
    return s[:, :k].to(lx.dtype), ids.gather(-1, pos).to(torch.int32)


def batch_norm(
    z: torch.Tensor,
    running_mean: torch.Tensor,
    running_var: torch.Tensor,
    training: bool,
    momentum: Optional[float] = BN_MOMENTUM,
    eps: float = BN_EPS,
    update: bool = True,
    num_batches_tracked: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``nn.BatchNorm1d(r, affine=False)`` on ``[T, r]`` (reference omni_moe.py:53-54,70-71).

    Train: batch mean and *biased* variance over the T rows normalise; the
    buffers move by ``momentum`` towards the batch mean and the *unbiased*
    variance.  Eval: the buffers normalise.  Statistics are fp32 whatever the
    storage dtype; the result is rounded once to z's dtype.  ``momentum=None`` is the
    module's cumulative moving average: the factor is 1 / (batches tracked so far + 1),
    read from ``num_batches_tracked`` (which the caller increments afterwards).  One sample
    in training raises, as the module does.
    """
    zf = z.float()
    if training:
        T = zf.size(0)
        if T == 1:
            raise ValueError(f"Expected more than 1 value per channel when training, got input size {tuple(z.shape)}")
        if momentum is None:
            momentum = 1.0 / (float(num_batches_tracked) + 1.0)
        mean = zf.mean(0)
        var = ((zf - mean) ** 2).mean(0)
        if update:
            unbiased = var * (T / max(T - 1, 1))
            running_mean.mul_(1 - momentum).add_(momentum * mean.to(running_mean.dtype))
            running_var.mul_(1 - momentum).add_(momentum * unbiased.to(running_var.dtype))
    else:
        mean, var = running_mean.float(), running_var.float()
    return ((zf - mean) * torch.rsqrt(var + eps)).to(z.dtype)


def log_softmax(l: torch.Tensor) -> torch.Tensor:
    """Row-wise log-softmax, fp32 inside, one rounding (reference omni_moe.py:77-78)."""
    lf = l.float()
    m = lf.max(-1, keepdim=True).values
    return (lf - m - torch.log(torch.exp(lf - m).sum(-1, keepdim=True))).to(l.dtype)


@dataclass
class BNState:
    """Buffers of one ``nn.BatchNorm1d(r, affine=False)``."""
    running_mean: torch.Tensor
    running_var: torch.Tensor
    num_batches_tracked: torch.Tensor

    @staticmethod
    def fresh(r: int) -> "BNState":
        return BNState(torch.zeros(r), torch.ones(r), torch.zeros((), dtype=torch.long))


def router_forward(
    x: torch.Tensor, wx: torch.Tensor, wy: torch.Tensor,
    bn_x: BNState, bn_y: BNState, top_k: int, training: bool, momentum: Optional[float] = BN_MOMENTUM,
):
    """Projection -> BN -> log-softmax -> select -> exp (reference omni_moe.py:147-178).

    Every stage rounds to x's dtype where torch would (Linear output, BN output,
    log-softmax output, candidate sums, exp).  Returns (gates, ids, scores).
    """
    r = wx.size(0)
    zx, zy = x @ wx.t(), x @ wy.t()
    nx = batch_norm(zx, bn_x.running_mean, bn_x.running_var, training, momentum, num_batches_tracked=bn_x.num_batches_tracked)
    ny = batch_norm(zy, bn_y.running_mean, bn_y.running_var, training, momentum, num_batches_tracked=bn_y.num_batches_tracked)
    if training:
        bn_x.num_batches_tracked += 1
        bn_y.num_batches_tracked += 1
    px, py = log_softmax(nx), log_softmax(ny)
    scores, ids = router_select(px, py, r, top_k)
    return torch.exp(scores.float()).to(x.dtype), ids, scores


# --------------------------------------------------------------------------
# expert-centric schedule
# --------------------------------------------------------------------------
def schedule(indices: torch.Tensor, num_experts: int):
    """(token, expert) pairs grouped by expert.

    Follows ``get_scheduling_info``'s tail part (reference omni_scheduler.py:48-101)
    in dense form: ``offsets[e]..offsets[e+1]`` bounds expert e's segment for ALL
    e in [0, N) (the reference compacts to the used experts, :79-87; the dense
    offsets carry the same segments).  ``sorted_pair_ids`` is the stable order
    (within a segment ascending pair id, i.e. ascending token); the reference's
    ``torch.sort`` (:71) leaves that order unspecified.
    Returns (offsets[N+1] int32, sorted_pair_ids[P] int32, sorted_token_ids[P] int32).
    """
    T, k = indices.shape
    flat = indices.reshape(-1).to(torch.int64)
    counts = torch.bincount(flat, minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    order = torch.sort(flat, stable=True).indices
    return offsets.to(torch.int32), order.to(torch.int32), (order // k).to(torch.int32)


# --------------------------------------------------------------------------
# atomic experts, shared MLP, layer
# --------------------------------------------------------------------------
def silu(x: torch.Tensor) -> torch.Tensor:
    """x*sigmoid(x) (reference activations.py:5-7)."""
    return x * torch.sigmoid(x)


def expert_forward(
    x: torch.Tensor, up: torch.Tensor, down: torch.Tensor,
    gates: torch.Tensor, indices: torch.Tensor, chunk: int = 2048,
    compute_dtype: Optional[torch.dtype] = torch.float32,
) -> torch.Tensor:
    """y[t] = sum_j silu(<x[t], U[id_tj]>) * g_tj * V[id_tj]  (reference omni_moe.py:181-189,
    tests/test_expert.py:8-25).  Token chunks bound the [chunk,k,H] gathers.

    ``compute_dtype=float32`` (default) evaluates the sums in fp32 from the stored
    values and rounds the result once to x's dtype; ``None`` keeps every torch op in
    x's dtype, reproducing the reference's intermediate roundings.
    """
    T, H = x.shape
    out = torch.empty_like(x)
    idx = indices.long()
    cd = compute_dtype or x.dtype
    for s in range(0, T, chunk):
        e = min(T, s + chunk)
        u = up[idx[s:e]].to(cd)                      # [c,k,H]
        v = down[idx[s:e]].to(cd)
        w = torch.matmul(u, x[s:e].to(cd).unsqueeze(-1)).squeeze(-1)   # [c,k]
        w = silu(w) * gates[s:e].to(cd)
        out[s:e] = torch.matmul(w.unsqueeze(-2), v).squeeze(-2).to(x.dtype)
    return out


def mlp_forward(x, wg, wu, wd) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)) with the rounding points of the reference op
    (interface.py:23-29, omni_mlp.py:53-61): the two projections round to x's dtype,
    the SwiGLU product is formed in fp32 and rounded once, then the down GEMM."""
    g = x @ wg.t()
    u = x @ wu.t()
    h = (silu(g.float()) * u.float()).to(x.dtype)
    return h @ wd.t()


@dataclass
class MoEWeights:
    """Parameters of the layer, by the reference's attribute names (omni_moe.py:42-58)."""
    gate_proj: torch.Tensor      # [I, H]
    up_proj: torch.Tensor        # [I, H]
    down_proj: torch.Tensor      # [H, I]
    router_gate_x: torch.Tensor  # [r, H]
    router_gate_y: torch.Tensor  # [r, H]
    up_embed: torch.Tensor       # [N, H]
    down_embed: torch.Tensor     # [N, H]


def moe_forward(
    hidden_states: torch.Tensor, w: MoEWeights, bn_x: BNState, bn_y: BNState,
    top_k: int, training: bool, expert_compute_dtype=torch.float32, momentum: Optional[float] = BN_MOMENTUM,
):
    """Whole layer (reference omni_moe.py:139-194).  Returns (y, gates, ids)."""
    shp = hidden_states.shape
    x = hidden_states.reshape(-1, shp[-1])
    gates, ids, _ = router_forward(x, w.router_gate_x, w.router_gate_y, bn_x, bn_y, top_k, training, momentum)
    e = expert_forward(x, w.up_embed, w.down_embed, gates, ids, compute_dtype=expert_compute_dtype)
    m = mlp_forward(x, w.gate_proj, w.up_proj, w.down_proj)
    return (m + e).reshape(shp), gates, ids


# --------------------------------------------------------------------------
# seeded synthetic inputs shared by tests, smoke and bench (CPU generator so the
# oracle and the device path see identical bits)
# --------------------------------------------------------------------------
def make_layer_inputs(seed: int, T: int, H: int, I: int, N: int, dtype=torch.bfloat16, w_std=0.02):
    g = torch.Generator().manual_seed(seed)
    r = math.floor(math.sqrt(N))
    n = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(dtype)
    x = n(1, T, H)
    w = MoEWeights(
        gate_proj=n(I, H, std=w_std), up_proj=n(I, H, std=w_std), down_proj=n(H, I, std=w_std),
        router_gate_x=n(r, H, std=w_std), router_gate_y=n(r, H, std=w_std),
        up_embed=n(N, H, std=w_std), down_embed=n(N, H, std=w_std),
    )
    return x, w


def make_expert_inputs(seed: int, T: int, H: int, N: int, k: int, dtype=torch.bfloat16, w_std=0.02):
    """x~N(0,1), tables~N(0,w_std), k distinct ids per token, gates = softmax(N(0,1))."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype)
    up = (torch.randn(N, H, generator=g) * w_std).to(dtype)
    down = (torch.randn(N, H, generator=g) * w_std).to(dtype)
    ids = torch.empty(T, k, dtype=torch.int32)
    for s in range(0, T, 4096):                       # argsort of uniforms = sample w/o replacement
        e = min(T, s + 4096)
        ids[s:e] = torch.rand(e - s, N, generator=g).argsort(-1)[:, :k].to(torch.int32)
    gates = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype)
    return x, up, down, gates, ids
