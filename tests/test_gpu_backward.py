"""GPU parity of the backward kernels (router, expert, SwiGLU) and of the trainable layer against
autograd of CPU restatements in fp64/fp32."""
import pytest
import torch

from oracle import omni_oracle as oracle

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
IDS = ["f32", "bf16", "f16"]


def _ops():
    from omni_moe.ops import hip
    return hip


def _tol(dtype):
    return {torch.float32: 2e-5, torch.bfloat16: 2e-2, torch.float16: 4e-3}[dtype]


def _close(got, want, dtype, what):
    """Compared on the scale of the expected tensor: gradients span orders of magnitude."""
    want = want.double().cpu()
    scale = max(want.abs().max().item(), 1e-30)
    err = (got.double().cpu() - want).abs().max().item() / scale
    assert err <= _tol(dtype), f"{what}: max error {err:.3e} of scale {scale:.3e}"


# ---------------------------------------------------------------- router
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("case", [(300, 64, 16), (128, 32, 8), (50, 512, 32), (64, 8, 64), (7, 1024, 128), (5, 4, 0)],
                         ids=lambda c: f"T{c[0]}-r{c[1]}-k{c[2]}")
def test_router_bwd_matches_scatter(case, dtype, device):
    """dlx[t, id // r] += ds, dly[t, id % r] += ds: against index_put_(accumulate) in fp64; fp32 is exact up to
    summation order."""
    T, r, k = case
    g = torch.Generator().manual_seed(T * 31 + r)
    ids = torch.randint(0, r * r, (T, k), generator=g, dtype=torch.int32)
    if k >= 4:
        ids[:, 1] = ids[:, 0]                                   # a repeated row coordinate and a repeated id
        ids[:, 3] = (ids[:, 2] // r) * r + (ids[:, 3] % r)
    ds = torch.randn(T, k, generator=g).to(dtype)
    print(f"router bwd T={T} r={r} k={k} {dtype}", flush=True)
    want_x = torch.zeros(T, r, dtype=torch.float64)
    want_y = torch.zeros(T, r, dtype=torch.float64)
    rows = torch.arange(T).unsqueeze(1).expand(T, k)
    want_x.index_put_((rows, (ids // r).long()), ds.double(), accumulate=True)
    want_y.index_put_((rows, (ids % r).long()), ds.double(), accumulate=True)
    dlx, dly = _ops().hip_omni_router_bwd_func(ds.to(device), ids.to(device), r)
    assert dlx.dtype == dtype and dlx.shape == (T, r)
    _close(dlx, want_x, dtype, "dlogits_x")
    _close(dly, want_y, dtype, "dlogits_y")


def test_router_func_autograd(device):
    """OmniRouterFunc end to end: scores come back differentiable, indices do not; gradients equal those of
    gathering the same ids out of the full outer sum."""
    T, r, k = 200, 32, 8
    g = torch.Generator().manual_seed(5)
    lx = torch.log_softmax(torch.randn(T, r, generator=g), -1)
    ly = torch.log_softmax(torch.randn(T, r, generator=g), -1)
    dlx, dly = lx.to(device).requires_grad_(), ly.to(device).requires_grad_()
    scores, idx = _ops().hip_omni_router_func(dlx, dly, r, k)
    assert scores.requires_grad and not idx.requires_grad
    w = torch.randn(T, k, generator=g)
    (scores * w.to(device)).sum().backward()
    cx, cy = lx.clone().requires_grad_(), ly.clone().requires_grad_()
    outer = (cx.unsqueeze(2) + cy.unsqueeze(1)).reshape(T, r * r)
    (outer.gather(1, idx.cpu().long()) * w).sum().backward()
    torch.testing.assert_close(dlx.grad.cpu(), cx.grad, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dly.grad.cpu(), cy.grad, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- experts
def _expert_reference(x, up, down, gates, ids, dy):
    """fp64 autograd of y[t] = sum_j silu(<x_t, U_e>) g_tj V_e in the gather form (reference tests/test_expert.py:8-25)."""
    x, up, down, gates = (t.double().clone().requires_grad_() for t in (x, up, down, gates))
    u, v = up[ids.long()], down[ids.long()]                        # [T,k,H]
    s = torch.einsum("th,tkh->tk", x, u)
    y = torch.einsum("tk,tkh->th", torch.nn.functional.silu(s) * gates, v)
    y.backward(dy.double())
    return y.detach(), x.grad, up.grad, down.grad, gates.grad


# the last case has 65 600 pairs over 50 experts: every segment crosses dozens of the weight pass's chunks
EXPERT_BWD_CASES = [(256, 1024, 512, 16), (300, 256, 64, 8), (64, 2048, 128, 4), (33, 96, 16, 6), (128, 4096, 32, 2), (16, 64, 1024, 32),
                    (4100, 64, 50, 16)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("case", EXPERT_BWD_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-N{c[2]}-k{c[3]}")
def test_expert_bwd_matches_autograd(case, dtype, device):
    T, H, N, k = case
    x, up, down, gates, ids = oracle.make_expert_inputs(11, T, H, N, k, dtype=dtype, w_std=0.05)
    g = torch.Generator().manual_seed(T + H)
    dy = torch.randn(T, H, generator=g).to(dtype)
    if k >= 2:
        ids[::3, 1] = ids[::3, 0]                                   # duplicate ids inside a token add up
    print(f"expert bwd T={T} H={H} N={N} k={k} {dtype}", flush=True)
    if H * x.element_size() > 8192:                                 # rows beyond 8 KiB: refused, as by the forward
        with pytest.raises(ValueError):
            _ops().hip_omni_expert_bwd_func(*(t.to(device) for t in (dy, x, up, down, gates, ids)))
        return
    _, wdx, wdu, wdv, wdg = _expert_reference(x, up, down, gates, ids, dy)
    dx, du, dv, dg = _ops().hip_omni_expert_bwd_func(*(t.to(device) for t in (dy, x, up, down, gates, ids)))
    for got, want, what in ((dx, wdx, "dx"), (du, wdu, "dup_weight"), (dv, wdv, "ddown_weight"), (dg, wdg, "drouting_weights")):
        assert got.dtype == dtype and got.shape == want.shape
        _close(got, want, dtype, what)
    # rows of experts nobody selected are exactly zero
    unused = torch.ones(N, dtype=torch.bool)
    unused[ids.long().flatten()] = False
    assert not du.cpu()[unused].any() and not dv.cpu()[unused].any()
    # and the result does not depend on the run
    again = _ops().hip_omni_expert_bwd_func(*(t.to(device) for t in (dy, x, up, down, gates, ids)))
    assert all(torch.equal(a, b) for a, b in zip((dx, du, dv, dg), again))


def test_expert_bwd_skewed_and_bad_ids(device):
    """One expert takes a third of all pairs (a long segment for a single wave); ids outside [0, N) contribute
    nothing to any gradient, as in the forward."""
    T, H, N, k = 512, 256, 64, 8
    x, up, down, gates, ids = oracle.make_expert_inputs(12, T, H, N, k, dtype=torch.float32, w_std=0.05)
    ids[:, :3] = 7
    ids[::5, 4] = N + 3
    ids[1::5, 5] = -1
    dy = torch.randn(T, H, generator=torch.Generator().manual_seed(1))
    ok = (ids >= 0) & (ids < N)
    _, wdx, wdu, wdv, wdg = _expert_reference(x, up, down, gates * ok, ids.clamp(0, N - 1), dy)
    dx, du, dv, dg = _ops().hip_omni_expert_bwd_func(*(t.to(device) for t in (dy, x, up, down, gates, ids)))
    _close(dx, wdx, torch.float32, "dx")
    _close(du, wdu, torch.float32, "dup_weight")
    _close(dv, wdv, torch.float32, "ddown_weight")
    _close(dg * ok.to(device), wdg * ok, torch.float32, "drouting_weights")
    assert not dg.cpu()[~ok].any()


def test_expert_func_autograd(device):
    T, H, N, k = 128, 256, 64, 8
    x, up, down, gates, ids = oracle.make_expert_inputs(13, T, H, N, k, dtype=torch.float32, w_std=0.05)
    leaves = [t.to(device).requires_grad_() for t in (x, up, down, gates)]
    y = _ops().hip_omni_expert_func(*leaves, ids.to(device))
    dy = torch.randn(T, H, generator=torch.Generator().manual_seed(2))
    y.backward(dy.to(device))
    wy, *wgrads = _expert_reference(x, up, down, gates, ids, dy)
    _close(y.detach(), wy, torch.float32, "y")
    for leaf, want, what in zip(leaves, wgrads, ("dx", "dup", "ddown", "dgates")):
        _close(leaf.grad, want, torch.float32, what)


# ---------------------------------------------------------------- SwiGLU and MLP
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_swiglu_fwd_bwd(dtype, device):
    g = torch.Generator().manual_seed(3)
    a, b, d = (torch.randn(77, 264, generator=g).to(dtype) * 3 for _ in range(3))
    ca, cb = a.double().requires_grad_(), b.double().requires_grad_()
    out = torch.nn.functional.silu(ca) * cb
    out.backward(d.double())
    hip = _ops()
    got = hip.hip_swiglu_func(a.to(device), b.to(device))
    _close(got, out.detach(), dtype, "swiglu")
    da, db = hip.hip_swiglu_bwd_func(d.to(device), a.to(device), b.to(device))
    _close(da, ca.grad, dtype, "dgate")
    _close(db, cb.grad, dtype, "dup")
    with pytest.raises(AssertionError):                       # as the reference's assert_omni_mlp_fwd_inputs (utils.py:68-78)
        hip.hip_swiglu_func(a.to(device), b.to(device)[:, :8])
    with pytest.raises(ValueError):
        hip.hip_swiglu_func(a.to(device), b.to(device).to(torch.float16 if dtype != torch.float16 else torch.float32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("shape", [(192, 128, 256), (4096, 1024, 4096), (77, 64, 136)], ids=lambda s: "T%d-H%d-I%d" % s)
def test_swiglu_linear_save_keeps_gate_and_up(shape, dtype, device):
    """The fused gate/up GEMM in its saving form (what the differentiable MLP op runs): gate and up are exactly the two
    plain projections, h is exactly the non-saving fused result."""
    from omni_moe.ops.hip import _lib
    from omni_moe.ops.hip.interface import OmniSwiGLULinearFunc
    T, H, I = shape
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, H, generator=g).to(dtype).to(device)
    wg = (torch.randn(I, H, generator=g) * 0.05).to(dtype).to(device)
    wu = (torch.randn(I, H, generator=g) * 0.05).to(dtype).to(device)
    hip = _ops()
    h = torch.empty(T, I, device=device, dtype=dtype)
    gate, up = torch.empty_like(h), torch.empty_like(h)
    code = _lib.load().omni_swiglu_linear_save_fwd(x.data_ptr(), wg.data_ptr(), wu.data_ptr(), h.data_ptr(), gate.data_ptr(), up.data_ptr(),
                                                   T, H, I, _lib.DTYPE_CODE[dtype], torch.cuda.current_stream().cuda_stream)
    assert code == 0
    assert torch.equal(gate, hip.hip_linear_func(x, wg))
    assert torch.equal(up, hip.hip_linear_func(x, wu))
    assert torch.equal(h, hip.hip_swiglu_linear_func(x, wg, wu))
    xr = x.clone().requires_grad_()
    assert torch.equal(OmniSwiGLULinearFunc.apply(xr, wg, wu), h)
    # fp32 storage and intermediate sizes that are not a multiple of 8 are refused (the Python op composes three launches there)
    assert _lib.load().omni_swiglu_linear_save_fwd(x.data_ptr(), wg.data_ptr(), wu.data_ptr(), h.data_ptr(), gate.data_ptr(), up.data_ptr(),
                                                   T, H, I, _lib.OMNI_F32, None) == _lib.ERR_UNSUPPORTED
    assert _lib.load().omni_swiglu_linear_save_fwd(x.data_ptr(), wg.data_ptr(), wu.data_ptr(), h.data_ptr(), gate.data_ptr(), up.data_ptr(),
                                                   T, H, I - 4, _lib.DTYPE_CODE[dtype], None) == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_mlp_func_autograd(dtype, device):
    """The differentiable MLP op (three GEMMs around the SwiGLU function) against fp64 autograd; its forward
    agrees with the fused inference path."""
    T, H, I = 192, 128, 256
    g = torch.Generator().manual_seed(4)
    x = torch.randn(T, H, generator=g).to(dtype)
    wg, wu = ((torch.randn(I, H, generator=g) * 0.1).to(dtype) for _ in range(2))
    wd = (torch.randn(H, I, generator=g) * 0.1).to(dtype)
    dy = torch.randn(T, H, generator=g).to(dtype)
    leaves = [t.to(device).requires_grad_() for t in (x, wg, wu, wd)]
    y = _ops().hip_omni_mlp_func(*leaves)
    y.backward(dy.to(device))
    cl = [t.double().requires_grad_() for t in (x, wg, wu, wd)]
    oracle.mlp_forward(*cl).backward(dy.double())
    _close(y.detach(), oracle.mlp_forward(*(t.double() for t in (x, wg, wu, wd))), dtype, "y")
    for leaf, c, what in zip(leaves, cl, ("dx", "dgate_weight", "dup_weight", "ddown_weight")):
        _close(leaf.grad, c.grad, dtype, what)
    with torch.no_grad():
        fused = _ops().hip_omni_mlp_func(*(t.detach() for t in leaves))
    _close(fused, y.detach(), dtype, "fused vs composed forward")


# ---------------------------------------------------------------- the layer trains
def _layer_pair(dtype, device, T=256, H=128, I=256, N=256, k=8, seed=6):
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    x, w = oracle.make_layer_inputs(seed, T, H, I, N, dtype=dtype, w_std=0.05)
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    layer.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                           "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
                           "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}, strict=False)
    return layer.to(device=device, dtype=dtype), x, w, k


@pytest.mark.parametrize("training", [True, False], ids=["train", "eval"])
def test_layer_backward_matches_oracle_autograd(training, device):
    """fp32 layer: forward and every parameter/input gradient against autograd through the CPU oracle, with the
    oracle fed the GPU's expert choice so that near-ties in the router cannot pick different experts."""
    layer, x, w, k = _layer_pair(torch.float32, device)
    layer.train(training)
    dx_in = x.to(device).requires_grad_()
    y = layer(dx_in)
    assert y.requires_grad
    dy = torch.randn(y.shape, generator=torch.Generator().manual_seed(8))
    y.backward(dy.to(device))

    names = ("gate_proj", "up_proj", "down_proj", "router_gate_x", "router_gate_y", "up_embed", "down_embed")
    cw = {n: getattr(w, n).double().requires_grad_() for n in names}
    cx = x.double().requires_grad_()
    xf = cx.view(-1, cx.size(-1))
    r = layer.num_expert_sqrt

    def half(weight):
        z = xf @ weight.t()
        if training:
            z = (z - z.mean(0)) / torch.sqrt(z.var(0, unbiased=False) + 1e-5)
        else:
            z = z / (1.0 + 1e-5) ** 0.5                               # fresh buffers: mean 0, var 1
        return torch.log_softmax(z, -1)

    lx, ly = half(cw["router_gate_x"]), half(cw["router_gate_y"])
    with torch.no_grad():
        _, ids = layer.eval().route(x.view(-1, x.size(-1)).to(device)) if not training else (None, None)
    if training:
        # the ids the GPU chose in this very forward: recompute them from the GPU's own log-probs path
        with torch.no_grad():
            fresh, *_ = _layer_pair(torch.float32, device)
            _, ids = fresh.train().route(x.view(-1, x.size(-1)).to(device))
    ids = ids.cpu().long()
    scores = (lx.unsqueeze(2) + ly.unsqueeze(1)).reshape(xf.size(0), r * r).gather(1, ids)
    gates = torch.exp(scores)
    e = torch.einsum("tk,tkh->th", torch.nn.functional.silu(torch.einsum("th,tkh->tk", xf, cw["up_embed"][ids])) * gates,
                     cw["down_embed"][ids])
    m = (torch.nn.functional.silu(xf @ cw["gate_proj"].t()) * (xf @ cw["up_proj"].t())) @ cw["down_proj"].t()
    want = (m + e).view_as(cx)
    want.backward(dy.double())

    _close(y.detach(), want.detach(), torch.float32, "y")
    tol = torch.float32
    _close(dx_in.grad, cx.grad, tol, "dx")
    for n in names:
        _close(getattr(layer, n).weight.grad, cw[n].grad, tol, f"d{n}")


def test_layer_trains_bf16(device):
    """A few SGD steps on a bf16 layer through the HIP forward and backward reduce a regression loss; the
    no_grad forward of the same weights takes the fused path and agrees with the composed one."""
    layer, x, w, k = _layer_pair(torch.bfloat16, device, seed=9)
    layer.train()
    xd = x.to(device)
    target = torch.randn(x.shape, generator=torch.Generator().manual_seed(10)).to(device=device, dtype=torch.bfloat16) * 0.1
    opt = torch.optim.SGD(layer.parameters(), lr=0.05)
    losses = []
    for _ in range(8):
        opt.zero_grad()
        loss = (layer(xd).float() - target.float()).pow(2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    print("losses", [round(v, 5) for v in losses], flush=True)
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in layer.parameters())
    assert losses[-1] < losses[0]
    layer.eval()
    composed = layer(xd).detach()
    with torch.no_grad():
        fused = layer(xd)
    torch.testing.assert_close(fused.float(), composed.float(), rtol=2e-2, atol=2e-2)


def test_backward_edge_cases(device):
    """No tokens, no slots: nothing to gather, weight gradients are all zero; argument errors are refused."""
    hip = _ops()
    H, N = 64, 32
    up, down = torch.randn(N, H, device=device), torch.randn(N, H, device=device)
    for T, k in ((0, 4), (5, 0)):
        x, dy = torch.randn(T, H, device=device), torch.randn(T, H, device=device)
        gates = torch.rand(T, k, device=device)
        ids = torch.zeros(T, k, dtype=torch.int32, device=device)
        dx, du, dv, dg = hip.hip_omni_expert_bwd_func(dy, x, up, down, gates, ids)
        assert dx.shape == (T, H) and dg.shape == (T, k)
        assert not du.any() and not dv.any() and not dx.any()
        dlx, dly = hip.hip_omni_router_bwd_func(torch.randn(T, k, device=device), ids, 8)
        assert dlx.shape == (T, 8) and not dlx.any() and not dly.any()
    with pytest.raises(ValueError):
        hip.hip_omni_expert_bwd_func(torch.randn(4, H + 8, device=device), torch.randn(4, H, device=device), up, down,
                                     torch.rand(4, 2, device=device), torch.zeros(4, 2, dtype=torch.int32, device=device))
    with pytest.raises(ValueError):
        hip.hip_omni_router_bwd_func(torch.randn(4, 2, device=device), torch.zeros(4, 3, dtype=torch.int32, device=device), 8)
    with pytest.raises(ValueError):                                   # r beyond what the kernel covers
        hip.hip_omni_router_bwd_func(torch.randn(4, 2, device=device), torch.zeros(4, 2, dtype=torch.int32, device=device), 2048)


@pytest.mark.parametrize("training", [True, False], ids=["train", "eval"])
@pytest.mark.parametrize("case", [(256, 128, 32, 8), (300, 64, 7, 6), (100, 96, 100, 16), (64, 64, 300, 32)],
                         ids=lambda c: f"T{c[0]}-H{c[1]}-r{c[2]}-k{c[3]}")
def test_router_stage_backward_matches_autograd(case, training, device):
    """OmniRouterStageFunc (projection, BatchNorm1d, log_softmax, router op, exp as one node) in fp32: gates and
    the gradients of x and both router weights against fp64 autograd of the same composition, evaluated at the
    ids the GPU selected."""
    T, H, r, k = case
    g = torch.Generator().manual_seed(T + r)
    x = torch.randn(T, H, generator=g)
    wx, wy = torch.randn(r, H, generator=g) * 0.2, torch.randn(r, H, generator=g) * 0.2
    run_mean, run_var = torch.randn(2, r, generator=g) * 0.1, torch.rand(2, r, generator=g) + 0.5
    w = torch.randn(T, k, generator=g)
    hip = _ops()
    leaves = [t.to(device).requires_grad_() for t in (x, wx, wy)]
    bufs = [t.to(device).clone() for t in (run_mean[0], run_var[0], run_mean[1], run_var[1])]
    nbt = [torch.zeros((), dtype=torch.long, device=device) for _ in range(2)]
    print(f"router stage T={T} H={H} r={r} k={k} training={training}", flush=True)
    gates, ids = hip.hip_omni_router_fwd_func(leaves[0], leaves[1], leaves[2], bufs[0], bufs[1], nbt[0], bufs[2], bufs[3], nbt[1],
                                              k, training=training)
    assert gates.requires_grad and not ids.requires_grad
    (gates * w.to(device)).sum().backward()

    cx, cwx, cwy = (t.double().requires_grad_() for t in (x, wx, wy))

    def half(weight, mean, var):
        z = cx @ weight.t()
        if training:
            z = (z - z.mean(0)) / torch.sqrt(z.var(0, unbiased=False) + 1e-5)
        else:
            z = (z - mean.double()) / torch.sqrt(var.double() + 1e-5)
        return torch.log_softmax(z, -1)

    lx, ly = half(cwx, run_mean[0], run_var[0]), half(cwy, run_mean[1], run_var[1])
    scores = (lx.unsqueeze(2) + ly.unsqueeze(1)).reshape(T, r * r).gather(1, ids.cpu().long())
    want = torch.exp(scores)
    (want * w.double()).sum().backward()
    _close(gates.detach(), want.detach(), torch.float32, "gates")
    for leaf, c, what in zip(leaves, (cx, cwx, cwy), ("dx", "dweight_x", "dweight_y")):
        assert torch.isfinite(leaf.grad).all()
        err = (leaf.grad.double().cpu() - c.grad).abs().max().item() / max(c.grad.abs().max().item(), 1e-30)
        assert err <= 2e-4, f"{what}: max error {err:.3e}"
    if training:
        assert nbt[0].item() == 1 and nbt[1].item() == 1


def test_expert_bwd_unused_rows_may_hold_nan(device):
    """As in the forward: the row that stands in for padded slots and out-of-range ids must not leak into any gradient."""
    T, H, N, k = 300, 256, 64, 6
    x, up, down, gates, ids = oracle.make_expert_inputs(14, T, H, N, k, dtype=torch.float32, w_std=0.05)
    ids = ids.clamp(min=1)
    ids[::9, 2] = N + 1
    dy = torch.randn(T, H, generator=torch.Generator().manual_seed(3))
    d = [t.to(device) for t in (dy, x, up, down, gates, ids)]
    want = _ops().hip_omni_expert_bwd_func(*d)
    up2, down2 = up.clone(), down.clone()
    up2[0], down2[0] = float("nan"), float("inf")
    got = _ops().hip_omni_expert_bwd_func(d[0], d[1], up2.to(device), down2.to(device), d[4], d[5])
    for a, b in zip(got, want):
        assert torch.isfinite(a).all() and torch.equal(a, b)
