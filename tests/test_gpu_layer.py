"""GPU parity of the MLP, the fused router and the whole OmniMoE layer against the CPU oracle."""
import pytest
import torch

from oracle import omni_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _inference():
    """These tests cover the fused forward; with autograd recording the module composes the
    differentiable operators instead (tests/test_gpu_backward.py)."""
    with torch.no_grad():
        yield


def _ops():
    from omni_moe.ops import hip
    return hip


# the first four are the reference's benchmark grid (tests/test_mlp.py:144-150): intermediate 1024 .. 65536
MLP_CASES = [(1024, 1024, 1024), (1024, 1024, 4096), (1024, 1024, 16384), (1024, 1024, 65536), (4096, 1024, 4096), (4100, 1024, 4096),
             (333, 256, 1000), (128, 64, 128), (512, 2048, 8192), (5, 8, 8),
             (8192, 128, 4096), (8200, 192, 2048)]      # streaming gate/up kernel with two and three K tiles per output tile, four tiles per block


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", MLP_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-I{c[2]}")
def test_mlp_matches_oracle(case, dtype, device):
    T, H, I = case
    g = torch.Generator().manual_seed(42)
    # reference benchmark distribution (tests/test_mlp.py:72-84): x~N(0,0.5), W~N(0,0.1) -- scaled
    # down for f16 at large I so the sums stay in range
    ws = 0.1 if dtype == torch.bfloat16 or I <= 1024 else 0.03
    x = (torch.randn(T, H, generator=g) * 0.5).to(dtype)
    wg, wu = ((torch.randn(I, H, generator=g) * ws).to(dtype) for _ in range(2))
    wd = (torch.randn(H, I, generator=g) * ws).to(dtype)
    res = torch.randn(T, H, generator=g).to(dtype)
    print(f"mlp T={T} H={H} I={I} {dtype}", flush=True)
    want = oracle.mlp_forward(x.float(), wg.float(), wu.float(), wd.float())      # fp32 everywhere
    d = [t.to(device) for t in (x, wg, wu, wd)]
    got = _ops().hip_omni_mlp_func(*d).cpu().float()
    scale = want.abs().max().item()
    # bf16 storage of gate/up/h contributes ~2^-8 relative noise per term; compare on the output's scale
    assert (got - want).abs().max().item() <= 2e-2 * max(scale, 1.0)
    torch.testing.assert_close(got / max(scale, 1.0), want / max(scale, 1.0), rtol=2e-2, atol=2e-2)
    got_r = _ops().hip_omni_mlp_func(*d, residual=res.to(device)).cpu().float()
    want_r = got.to(dtype).float() + res.float()
    torch.testing.assert_close(got_r, want_r.to(dtype).float(), rtol=1e-2, atol=1e-2 * max(scale, 1.0))


@pytest.mark.parametrize("case", [(512, 256, 1024), (300, 100, 260), (64, 1024, 512)], ids=lambda c: f"T{c[0]}-H{c[1]}-I{c[2]}")
def test_mlp_fp32_matches_oracle(case, device):
    T, H, I = case
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, H, generator=g)
    wg, wu, wd = torch.randn(I, H, generator=g) * 0.05, torch.randn(I, H, generator=g) * 0.05, torch.randn(H, I, generator=g) * 0.05
    res = torch.randn(T, H, generator=g)
    print(f"mlp fp32 T={T} H={H} I={I}", flush=True)
    want = oracle.mlp_forward(x.double(), wg.double(), wu.double(), wd.double()).float()
    d = [t.to(device) for t in (x, wg, wu, wd)]
    got = _ops().hip_omni_mlp_func(*d).cpu()
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5 * max(1.0, want.abs().max().item()))
    got_r = _ops().hip_omni_mlp_func(*d, residual=res.to(device)).cpu()
    torch.testing.assert_close(got_r, want + res, rtol=1e-4, atol=1e-5 * max(1.0, want.abs().max().item()))


# the last two make the projection GEMM pick its 128 x 128 and 256 x 256 tiles (statistics epilogue included)
ROUTER_FWD_CASES = [(4096, 1024, 64, 16), (1024, 256, 32, 8), (2048, 2048, 512, 32), (300, 520, 36, 10), (300, 576, 36, 10),
                    (4096, 256, 512, 32), (16384, 256, 512, 32), (200, 128, 1300, 16)]      # last: more than 1024 keys per half


def _bn_buffers(r, dtype, device=None):
    m, v = torch.zeros(r, dtype=dtype), torch.ones(r, dtype=dtype)
    n = torch.zeros((), dtype=torch.long)
    return [t.to(device) if device else t for t in (m, v, n)]


@pytest.mark.parametrize("training", [True, False], ids=["train", "eval"])
@pytest.mark.parametrize("case", ROUTER_FWD_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-r{c[2]}-k{c[3]}")
def test_router_fwd_matches_oracle(case, training, device):
    T, H, r, k = case
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=g).to(dtype)
    wx, wy = ((torch.randn(r, H, generator=g) / H ** 0.5).to(dtype) for _ in range(2))
    bx, by = oracle.BNState.fresh(r), oracle.BNState.fresh(r)
    if not training:   # eval: give the buffers content (a per-key bias and scale)
        for b in (bx, by):
            b.running_mean.copy_(torch.randn(r, generator=g) * 0.3)
            b.running_var.copy_(torch.rand(r, generator=g) + 0.5)
    dbx = [bx.running_mean.clone().to(device), bx.running_var.clone().to(device), torch.zeros((), dtype=torch.long, device=device)]
    dby = [by.running_mean.clone().to(device), by.running_var.clone().to(device), torch.zeros((), dtype=torch.long, device=device)]
    print(f"router_fwd T={T} H={H} r={r} k={k} training={training}", flush=True)
    want_g, want_i, want_s = oracle.router_forward(x, wx, wy, bx, by, k, training)
    got_g, got_i, got_s = _ops().hip_omni_router_fwd_func(x.to(device), wx.to(device), wy.to(device), *dbx, *dby, k,
                                                          training=training, return_scores=True)
    torch.cuda.synchronize()
    got_i, got_g, got_s = got_i.cpu(), got_g.cpu(), got_s.cpu()
    # internal consistency, exact: the gate is exp of the score, scores descend
    assert torch.equal(got_g.float(), torch.exp(got_s.float()).to(dtype).float())
    assert (got_s[:, :-1].float() >= got_s[:, 1:].float()).all()
    # end-to-end index agreement with the oracle (the projections differ in fp32 summation
    # order, so a bf16 rounding can flip): >= 99.9 % of the per-token expert sets
    same_pos = (got_i == want_i).float().mean().item()
    a, b = got_i.sort(-1).values, want_i.sort(-1).values
    set_agree = (a == b).float().mean().item()
    print(f"   position agreement {same_pos:.5f}, set agreement {set_agree:.5f}")
    assert set_agree >= 0.999, set_agree
    assert same_pos >= 0.99, same_pos
    torch.testing.assert_close(got_g.float(), want_g.float(), rtol=2e-2, atol=2e-2)
    # running statistics
    if training:
        torch.testing.assert_close(dbx[0].cpu(), bx.running_mean, rtol=1e-3, atol=1e-4)
        torch.testing.assert_close(dbx[1].cpu(), bx.running_var, rtol=1e-3, atol=1e-4)
        torch.testing.assert_close(dby[1].cpu(), by.running_var, rtol=1e-3, atol=1e-4)
        assert dbx[2].item() == 1 and dby[2].item() == 1
    else:
        assert torch.equal(dbx[0].cpu(), bx.running_mean) and dbx[2].item() == 0


def test_router_fwd_select_is_exact_given_same_logprobs(device):
    """Feeding the oracle's selection the device's own scores must reproduce the device's ids
    bit for bit: run the fused router, rebuild the log-probs it saw from its z, compare."""
    T, H, r, k = 1024, 512, 64, 16
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, generator=g).bfloat16()
    wx, wy = ((torch.randn(r, H, generator=g) / H ** 0.5).bfloat16() for _ in range(2))
    hip = _ops()
    z = hip.hip_linear_func(x.to(device), torch.cat([wx, wy]).to(device)).cpu()       # same GEMM kernel
    bx, by = oracle.BNState.fresh(r), oracle.BNState.fresh(r)
    px = oracle.log_softmax(oracle.batch_norm(z[:, :r].contiguous(), bx.running_mean, bx.running_var, True))
    py = oracle.log_softmax(oracle.batch_norm(z[:, r:].contiguous(), by.running_mean, by.running_var, True))
    want_s, want_i = oracle.router_select(px, py, r, k)
    d = _bn_buffers(r, torch.float32, device) + _bn_buffers(r, torch.float32, device)
    _, got_i, got_s = hip.hip_omni_router_fwd_func(x.to(device), wx.to(device), wy.to(device), *d, k, training=True, return_scores=True)
    agree = (got_i.cpu() == want_i).float().mean().item()
    print(f"   agreement given device z: {agree:.6f}")
    assert agree >= 0.9995          # only exp/log ulp differences between host and device libm remain


LAYER_CASES = [
    # (T, H, I, N, k, seed)
    (96, 8192, 256, 64, 4, 5),         # expert rows of 16 KiB: the split kernels in two column blocks
    (512, 256, 1024, 1024, 8, 0),      # benchmark config 1 shape, in bf16
    (4096, 1024, 4096, 4096, 16, 3),   # benchmark config 4 (README shape)
    (300, 128, 256, 1000, 8, 1),       # N not a square: r = floor(sqrt(N)) = 31 (omni_moe.py:38), odd, ids < 961
    (300, 128, 256, 1000, 40, 1),      # and k > r, so k' = r
    (64, 64, 128, 50, 6, 2),           # r = 7
    (200, 64, 128, 1100 * 1100, 8, 4), # r = 1100: more keys per half than the select kernels hold in registers
]


@pytest.mark.parametrize("training", [True, False], ids=["train", "eval"])
@pytest.mark.parametrize("case", LAYER_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-I{c[2]}-N{c[3]}-k{c[4]}")
def test_layer_matches_oracle(case, training, device):
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    T, H, I, N, k, seed = case
    x, w = oracle.make_layer_inputs(seed, T, H, I, N)
    r = w.router_gate_x.size(0)
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    sd = {"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
          "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
          "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}
    missing, unexpected = layer.load_state_dict(sd, strict=False)
    assert not unexpected and all("router_norm" in m for m in missing)
    layer = layer.to(device=device, dtype=torch.bfloat16)
    layer.train(training)
    print(f"layer T={T} H={H} I={I} N={N} k={k} training={training}", flush=True)
    bx, by = oracle.BNState.fresh(r), oracle.BNState.fresh(r)
    want, want_g, want_i = oracle.moe_forward(x, w, bx, by, k, training)
    got = layer(x.to(device))
    torch.cuda.synchronize()
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    got_g, got_i = layer.eval().route(x.view(-1, H).to(device)) if not training else (None, None)
    # tokens whose expert set matches the oracle's must match in value; the others differ by
    # which near-tied expert was picked, which changes y by at most a few gate*|V| -- still small
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=2e-2, atol=2e-2)
    # the same bound on the scale of the output (|y| is a few 0.01 at these weights, where a flat 2e-2 says little)
    scale = want.float().abs().max().item()
    assert (got.cpu().float() - want.float()).abs().max().item() <= 2e-2 * scale, scale
    if training:
        assert layer.router_norm_x.num_batches_tracked.item() == 1
        torch.testing.assert_close(layer.router_norm_x.running_mean.float().cpu(), bx.running_mean, rtol=2e-2, atol=2e-3)
    else:
        set_agree = (got_i.cpu().sort(-1).values == want_i.sort(-1).values).float().mean().item()
        print(f"   expert-set agreement {set_agree:.5f}")
        assert set_agree >= 0.999


@pytest.mark.parametrize("training", [True, False], ids=["train", "eval"])
def test_layer_config1_fp32(training, device):
    """benchmark config 1, the reference's CPU-runnable case, at full size in fp32:
    1 x 512 tokens, hidden 256, intermediate 1024, 1024 experts (32 x 32), top-8, seed 0."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    T, H, I, N, k = 512, 256, 1024, 1024, 8
    x, w = oracle.make_layer_inputs(0, T, H, I, N, dtype=torch.float32)
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    layer.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                           "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
                           "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}, strict=False)
    layer = layer.to(device).train(training)
    bx, by = oracle.BNState.fresh(32), oracle.BNState.fresh(32)
    print(f"layer config 1 fp32 training={training}", flush=True)
    want, want_g, want_i = oracle.moe_forward(x, w, bx, by, k, training)
    got = layer(x.to(device))
    torch.cuda.synchronize()
    assert got.dtype == torch.float32
    layer.eval()
    if training:   # route again with the updated buffers on both sides
        want_g, want_i, _ = oracle.router_forward(x.view(-1, H), w.router_gate_x, w.router_gate_y, bx, by, k, False)
    got_g, got_i = layer.route(x.view(-1, H).to(device))
    # fp32 scores: ties practically never occur, so the ids are forced up to fp32 summation order
    set_agree = (got_i.cpu().sort(-1).values == want_i.sort(-1).values).all(-1).float().mean().item()
    print(f"   tokens with identical expert sets: {set_agree:.5f}")
    assert set_agree >= 0.999
    torch.testing.assert_close(got_g.cpu(), want_g, rtol=1e-3, atol=1e-6)
    same = (got_i.cpu().sort(-1).values == want_i.sort(-1).values).all(-1) if not training else torch.ones(T, dtype=torch.bool)
    torch.testing.assert_close(got.cpu().view(-1, H)[same], want.view(-1, H)[same], rtol=1e-3, atol=2e-5)
    if training:
        torch.testing.assert_close(layer.router_norm_x.running_mean.cpu(), bx.running_mean, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(layer.router_norm_y.running_var.cpu(), by.running_var, rtol=1e-4, atol=1e-6)


def test_layer_config5_large_skewed(device):
    """benchmark config 5: 8 x 4096 tokens, hidden 2048, intermediate 8192, 262144 experts
    (512 x 512 keys), top-32, bf16, router key popularity ~ Zipf(1.1), seed 4.

    The reference's router has no bias (omni_moe.py:47-52), so the per-key bias b_i = -1.1*ln(1+i)
    enters through eval-mode BatchNorm buffers: running_mean = -b, running_var = 1 - eps.  The whole
    batch runs on the GPU; the oracle checks a token subset (eval mode is token-independent) and the
    schedule of all 1M pairs."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    T, H, I, N, k, r = 32768, 2048, 8192, 262144, 32, 512
    g = torch.Generator().manual_seed(4)
    n = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).bfloat16()
    x = n(8, 4096, H)
    w = oracle.MoEWeights(gate_proj=n(I, H, std=0.02), up_proj=n(I, H, std=0.02), down_proj=n(H, I, std=0.02),
                          router_gate_x=n(r, H, std=0.02), router_gate_y=n(r, H, std=0.02),
                          up_embed=n(N, H, std=0.02), down_embed=n(N, H, std=0.02))
    bias = -1.1 * torch.log1p(torch.arange(r, dtype=torch.float32))
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    layer.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                           "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
                           "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}, strict=False)
    for bn in (layer.router_norm_x, layer.router_norm_y):
        bn.running_mean.copy_(-bias)
        bn.running_var.fill_(1.0 - bn.eps)
    layer = layer.to(device=device, dtype=torch.bfloat16).eval()
    print("layer config 5: 32768 tokens, 262144 experts, top-32", flush=True)
    y = layer(x.to(device))
    gates, ids = layer.route(x.view(-1, H).to(device))
    torch.cuda.synchronize()
    assert y.shape == x.shape and torch.isfinite(y.float()).all()
    # at this size the module keeps to one stream (the GEMMs then take their streaming form); the two-stream schedule, with
    # the other GEMM kernels and the add as a kernel of its own, must give the same bits
    layer.overlap_max_work = 2 ** 62
    assert torch.equal(layer(x.to(device)), y)
    del layer.overlap_max_work
    # schedule of the real, skewed assignment: offsets exact, pairs a grouped permutation
    sched = _ops().hip_omni_schedule_func(ids, N)
    ids_c = ids.cpu()
    want_off, want_pairs, _ = oracle.schedule(ids_c, N)
    assert torch.equal(sched.offsets.cpu(), want_off)
    assert torch.equal(sched.sorted_pair_ids.cpu(), want_pairs)
    seg = (want_off[1:] - want_off[:-1]).float()
    print(f"   pairs per expert: max {int(seg.max())}, mean over used {seg[seg > 0].mean():.1f}, used experts {int((seg > 0).sum())}")
    assert seg.max() > 100 * seg[seg > 0].mean()          # the skew is there
    # oracle on a token subset (buffers as the bf16 module holds them)
    sub = torch.arange(0, T, 128)
    bx = oracle.BNState(layer.router_norm_x.running_mean.float().cpu(), layer.router_norm_x.running_var.float().cpu(), torch.zeros((), dtype=torch.long))
    by = oracle.BNState(layer.router_norm_y.running_mean.float().cpu(), layer.router_norm_y.running_var.float().cpu(), torch.zeros((), dtype=torch.long))
    xs = x.view(-1, H)[sub].unsqueeze(0)
    want, want_g, want_i = oracle.moe_forward(xs, w, bx, by, k, training=False)
    got_i = ids_c[sub]
    set_agree = (got_i.sort(-1).values == want_i.sort(-1).values).float().mean().item()
    print(f"   expert-set agreement on {len(sub)} tokens: {set_agree:.5f}")
    assert set_agree >= 0.999
    torch.testing.assert_close(y.view(-1, H)[sub.to(device)].float().cpu(), want.view(-1, H).float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(gates.cpu()[sub].float(), want_g.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("training", [False, True], ids=["eval", "train"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("two_streams", [False, True], ids=["one-stream", "two-streams"])
def test_layer_expert_term_visible_auto_split(two_streams, dtype, training, device):
    """A layer whose expert branch is as large as its MLP branch (weights ~ N(0, 0.1)) and whose shape makes the layer call
    pick the hidden-split expert algorithm (4096 tokens x 32 = 131072 pairs, tables that overflow one L2): y - mlp must equal
    the oracle's expert term on the expert term's own scale, on one stream and on two.  A layer that dropped or mis-wired
    router -> experts (wrong gates or ids buffer, workspace overlap, missing join) fails here.  In training mode the router
    normalises with the statistics of the whole 4096-token batch, on the device and in the oracle."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    T, H, I, N, k = 4096, 512, 512, (1024 if dtype == torch.float32 else 4096), 32
    x, w = oracle.make_layer_inputs(21, T, H, I, N, dtype=dtype, w_std=0.1)
    # the shared MLP scaled down to the size of the expert term (batch statistics flatten the gates: smaller still in training)
    w.down_proj = (w.down_proj.float() * (0.006 if training else 0.03)).to(dtype)
    r = w.router_gate_x.size(0)
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    layer.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                           "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
                           "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}, strict=False)
    layer = layer.to(device=device, dtype=dtype).train(training)
    layer.overlap_branches = two_streams
    layer.overlap_min_work = 0
    from omni_moe.ops.hip import _lib
    lib = _lib.load()
    es = 4 if dtype == torch.float32 else 2
    assert lib.omni_expert_workspace_bytes(T, H, N, k, _lib.DTYPE_CODE[dtype], _lib.ALGO_AUTO) == 8 * T * k * 4, "AUTO should pick the split algorithm here"
    print(f"layer with visible expert term, {dtype}, two_streams={two_streams}, training={training}", flush=True)
    xd = x.to(device)
    y = layer(xd).view(-1, H)
    mlp = _ops().hip_omni_mlp_func(xd.view(-1, H), layer.gate_proj.weight, layer.up_proj.weight, layer.down_proj.weight)
    gates, ids = layer.route(xd.view(-1, H))               # training: the same batch again, so the same statistics and ids
    torch.cuda.synchronize()
    bx, by = oracle.BNState.fresh(r), oracle.BNState.fresh(r)
    want_y, want_g, want_i = oracle.moe_forward(x, w, bx, by, k, training=training)
    if training:
        assert layer.router_norm_x.num_batches_tracked.item() == 2
    # the oracle's expert term for the ids the device chose (near-tied scores may resolve differently in bf16)
    want_e = oracle.expert_forward(x.view(-1, H), w.up_embed, w.down_embed, gates.cpu(), ids.cpu()).float()
    e_scale, m_scale = want_e.abs().max().item(), mlp.float().abs().max().item()
    print(f"   max |experts| {e_scale:.3f}, max |mlp| {m_scale:.3f}")
    assert e_scale > 0.15 * m_scale                            # the expert term is visible (batch statistics spread the gates a little thinner)
    got_e = (y.float() - mlp.float()).cpu()
    tol = 1e-4 if dtype == torch.float32 else 2e-2            # bf16: y and mlp are rounded to bf16 on the scale of their sum
    assert (got_e - want_e).abs().max().item() <= tol * (e_scale + m_scale), (got_e - want_e).abs().max().item()
    assert (got_e - want_e).abs().mean().item() <= 0.1 * tol * (e_scale + m_scale)
    same = (ids.cpu().sort(-1).values == want_i.sort(-1).values).all(-1)
    assert same.float().mean().item() >= (0.999 if dtype == torch.float32 else 0.97)
    torch.testing.assert_close(y.cpu().float()[same], want_y.view(-1, H).float()[same], rtol=tol, atol=tol * (e_scale + m_scale))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_layer_two_streams_equals_one_stream(dtype, device):
    """The two-stream schedule (router+experts beside the MLP, joined by omni_add_inplace) and the
    one-stream schedule (add fused into the down projection) give bit-identical output, call after call."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    torch.manual_seed(0)
    layer = OmniMoE(OmniMoEConfig(256, 512, "silu", 1024, 8)).to(device=device, dtype=dtype).eval()
    layer.overlap_min_work = 0                    # two streams whatever the size
    x = torch.randn(3, 100, 256, device=device).to(dtype)
    layer.overlap_branches = False
    ref = layer(x)
    layer.overlap_branches = True
    for _ in range(5):
        assert torch.equal(layer(x), ref)
    # and next to other work on the caller's stream
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        z = x * 2
        out = layer(z)
    s.synchronize()
    layer.overlap_branches = False
    assert torch.equal(out, layer(x * 2))


def test_layer_copies_and_saves_like_a_plain_module(device, tmp_path):
    """After a two-stream forward (side stream and events in use) a layer is still a plain nn.Module:
    copy.deepcopy, torch.save / torch.load and a state_dict round trip give layers with identical output."""
    import copy
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    torch.manual_seed(3)
    cfg = OmniMoEConfig(256, 512, "silu", 1024, 8)
    layer = OmniMoE(cfg).to(device=device, dtype=torch.bfloat16).eval()
    layer.overlap_min_work = 0
    x = torch.randn(2, 200, 256, device=device).bfloat16()
    want = layer(x)
    twin = copy.deepcopy(layer)
    assert torch.equal(twin(x), want)
    path = str(tmp_path / "layer.pt")
    torch.save(layer, path)
    loaded = torch.load(path, weights_only=False)           # a file this test wrote itself
    assert torch.equal(loaded(x), want)
    fresh = OmniMoE(cfg).to(device=device, dtype=torch.bfloat16).eval()
    fresh.load_state_dict(layer.state_dict())
    fresh.overlap_min_work = 0
    assert torch.equal(fresh(x), want)
    assert not any(isinstance(v, (torch.cuda.Stream, torch.cuda.Event)) for v in vars(layer).values())


def test_layer_takes_noncontiguous_weights(device):
    """The reference's operators make every tensor argument contiguous (utils.py:47-65); the fused layer call does too."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    torch.manual_seed(4)
    layer = OmniMoE(OmniMoEConfig(128, 256, "silu", 256, 8)).to(device=device, dtype=torch.bfloat16).eval()
    x = torch.randn(1, 300, 128, device=device).bfloat16()
    want = layer(x)
    w = layer.down_proj.weight.data
    layer.down_proj.weight.data = w.t().contiguous().t()    # same values, column-major storage
    assert not layer.down_proj.weight.is_contiguous()
    assert torch.equal(layer(x), want)


def test_add_inplace(device):
    hip = _ops()
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        a, b = torch.randn(37, 64, device=device).to(dtype), torch.randn(37, 64, device=device).to(dtype)
        want = (a.float() + b.float()).to(dtype)
        assert torch.equal(hip.hip_add_inplace_func(a.clone(), b), want)
    with pytest.raises(ValueError):
        hip.hip_add_inplace_func(torch.zeros(4, 8, device=device), torch.zeros(4, 9, device=device))


# (M, N, K): the first five select the 128 x 128 output tiles (too few 256 x 256 tiles to fill the chip), ragged M
# included; then a big-tile case, N % 8 == 4 (rows written 8 bytes per lane instead of 16), a ragged last column tile
LINEAR_CASES = [(3300, 1024, 512), (3300, 1024, 640), (3300, 1024, 576), (4096, 1024, 4096), (2049, 1536, 1024),
                (4096, 4096, 256), (300, 100, 264), (333, 1000, 256), (70, 4, 8),
                (300, 62, 128), (129, 1001, 64), (70, 6, 16), (5, 1, 8),       # N % 4 != 0: element-wise stores
                # few 64 x 64 tiles and K >= 512: the K tiles of a block dealt out over its waves (even and ragged shares, tails)
                (4096, 128, 1024), (1000, 104, 512), (130, 72, 640), (64, 64, 4096), (200, 6, 576), (33, 250, 832),
                # the streaming form with a ragged last row tile and with tile counts that are no whole rounds of 256
                (4100, 4096, 512), (3328, 4096, 512), (4353, 4096, 128)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", LINEAR_CASES, ids=lambda c: f"M{c[0]}-N{c[1]}-K{c[2]}")
def test_linear_matches_matmul(case, dtype, device):
    """y = x W^T (+ residual) against an fp64 matmul, over the tile shapes and both store widths."""
    M, N, K = case
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    res = torch.randn(M, N, generator=g).to(dtype)
    print(f"linear M={M} N={N} K={K} {dtype}", flush=True)
    want = x.double() @ w.double().t()
    got = _ops().hip_linear_func(x.to(device), w.to(device)).cpu()
    # one rounding of an fp32 sum: half an ulp of the storage dtype plus fp32 summation noise
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    err = (got.double() - want).abs()
    assert (err <= ulp * want.abs() * 1.01 + 1e-4 * want.abs().max()).all()
    got_r = _ops().hip_linear_func(x.to(device), w.to(device), residual=res.to(device)).cpu()
    assert torch.equal(got_r, (got.float() + res.float()).to(dtype))


# (M, columns per weight matrix, K): streaming kernel (second matrix = whole tiles), K tiles dealt out over the waves, ring kernel, staged kernel
LINEAR2_CASES = [(8192, 512, 256), (16384, 256, 128), (1000, 52, 512), (3000, 200, 192), (300, 36, 40)]


@pytest.mark.parametrize("case", LINEAR2_CASES, ids=lambda c: f"M{c[0]}-N2x{c[1]}-K{c[2]}")
def test_linear_two_weight_matrices_equals_one(case, device):
    """omni_linear2_fwd (the router projection's form: the upper half of the output columns comes from a second weight
    matrix) gives bit for bit what omni_linear_fwd gives on the concatenated weights."""
    from omni_moe.ops.hip import _lib
    M, n, K = case
    g = torch.Generator().manual_seed(M + n)
    x = torch.randn(M, K, generator=g).bfloat16().to(device)
    w_lo = (torch.randn(n, K, generator=g) * 0.05).bfloat16().to(device)
    w_hi = (torch.randn(n, K, generator=g) * 0.05).bfloat16().to(device)
    print(f"linear2 M={M} N=2x{n} K={K}", flush=True)
    want = _ops().hip_linear_func(x, torch.cat([w_lo, w_hi], 0))
    ref = (x.double() @ torch.cat([w_lo, w_hi], 0).double().t())
    assert ((want.double() - ref).abs() <= 2.0 ** -8 * ref.abs() * 1.01 + 1e-4 * ref.abs().max()).all()
    got = torch.empty(M, 2 * n, dtype=torch.bfloat16, device=device)
    lib = _lib.load()
    _lib.check(lib.omni_linear2_fwd(x.data_ptr(), w_lo.data_ptr(), w_hi.data_ptr(), got.data_ptr(), M, K, n,
                                    _lib.DTYPE_CODE[torch.bfloat16], _lib.stream_ptr()), "omni_linear2_fwd")
    torch.cuda.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("overlap", [True, False], ids=["two-streams", "one-stream"])
def test_layer_is_graph_capturable(overlap, device):
    """The library only launches kernels and records/waits events, so a whole layer forward (fork and join
    included) can be captured into a HIP graph; every replay, with eager work in between, equals the eager result."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    torch.manual_seed(1)
    layer = OmniMoE(OmniMoEConfig(256, 512, "silu", 1024, 8)).to(device=device, dtype=torch.bfloat16).eval()
    layer.overlap_branches = overlap
    layer.overlap_min_work = 0
    x = torch.randn(2, 150, 256, device=device).bfloat16()
    want = layer(x).clone()
    warm = torch.cuda.Stream()
    warm.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(warm):
        layer(x)
    torch.cuda.current_stream().wait_stream(warm)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = layer(x)
    for _ in range(4):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
        assert torch.equal(layer(x * 0.5), layer(x * 0.5))      # eager work between the replays
        torch.cuda.synchronize()


def test_layer_cumulative_batch_norm(device):
    """router_norm_x/y with momentum=None (cumulative moving average, factor 1 / num_batches_tracked): three training
    steps on different batches leave the buffers the oracle predicts, counters included."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    T, H, I, N, k = 300, 128, 256, 256, 8
    _, w = oracle.make_layer_inputs(9, T, H, I, N, dtype=torch.float32)
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    layer.router_norm_x.momentum = layer.router_norm_y.momentum = None
    layer.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                           "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
                           "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}, strict=False)
    layer = layer.to(device).train()
    bx, by = oracle.BNState.fresh(16), oracle.BNState.fresh(16)
    g = torch.Generator().manual_seed(10)
    for step in range(3):
        x = torch.randn(1, T, H, generator=g) * (1.0 + step)
        want, _, _ = oracle.moe_forward(x, w, bx, by, k, training=True, momentum=None)
        got = layer(x.to(device))
        assert layer.router_norm_x.num_batches_tracked.item() == step + 1 == int(bx.num_batches_tracked)
        torch.testing.assert_close(layer.router_norm_x.running_mean.cpu(), bx.running_mean, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(layer.router_norm_y.running_var.cpu(), by.running_var, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4)
    layer.router_norm_y.momentum = 0.1
    with pytest.raises(ValueError):                               # one momentum for both halves
        layer(x.to(device))


@pytest.mark.parametrize("training", [True, False], ids=["train", "eval"])
@pytest.mark.parametrize("T", [1, 2, 3, 5, 31, 33, 65])
def test_layer_tiny_token_counts(T, training, device):
    """A handful of tokens (one wave, one partial strip, a single BatchNorm sample in training), on one and on two
    streams: same tolerance as the big cases, and both schedules bit-identical."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    H, I, N, k = 128, 256, 256, 8
    x, w = oracle.make_layer_inputs(T, T, H, I, N)
    sd = {"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
          "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
          "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}
    if T == 1 and training:
        # batch statistics of a single sample: nn.BatchNorm1d raises (reference omni_moe.py:70-71), and so do the oracle and the layer
        with pytest.raises(ValueError):
            oracle.moe_forward(x, w, oracle.BNState.fresh(16), oracle.BNState.fresh(16), k, training)
        for overlap in (True, False):
            layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
            layer.load_state_dict(sd, strict=False)
            layer = layer.to(device=device, dtype=torch.bfloat16).train()
            layer.overlap_branches = overlap
            layer.overlap_min_work = 0
            with pytest.raises(ValueError, match="more than 1 value per channel"):
                layer(x.to(device))
            assert layer.router_norm_x.num_batches_tracked.item() == 0
        return
    want, _, _ = oracle.moe_forward(x, w, oracle.BNState.fresh(16), oracle.BNState.fresh(16), k, training)
    outs = []
    for overlap in (True, False):
        layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
        layer.load_state_dict(sd, strict=False)
        layer = layer.to(device=device, dtype=torch.bfloat16).train(training)
        layer.overlap_branches = overlap
        layer.overlap_min_work = 0
        outs.append(layer(x.to(device)))
    torch.testing.assert_close(outs[0].cpu().float(), want.float(), rtol=2e-2, atol=2e-2)
    assert torch.equal(outs[0], outs[1])
