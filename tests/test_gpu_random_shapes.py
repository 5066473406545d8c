"""Seeded sweeps over many small, odd shapes, one process: the integer/index paths stay bit-exact against the oracle,
the floating-point ones inside their tolerance.  Shapes a hand-picked list would not think of."""
import random

import pytest
import torch

from oracle import omni_oracle as oracle

pytestmark = pytest.mark.gpu


def _ops():
    from omni_moe.ops import hip
    return hip


def test_router_select_random_shapes(device):
    rng = random.Random(1234)
    hip = _ops()
    for case in range(60):
        r = rng.choice([2, 3, 5, 8, 13, 31, 64, 65, 100, 127, 128, 129, 200, 257])
        kmax = min(128, r * r)
        k = 2 * rng.randint(1, kmax // 2)
        T = rng.choice([1, 2, 7, 63, 64, 65, 130, 257])
        dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        g = torch.Generator().manual_seed(case)
        if rng.random() < 0.5:                     # coarse grid: plenty of ties in the halves and among the sums
            lx = (torch.randint(-8, 1, (T, r), generator=g).float() / 4).to(dtype)
            ly = (torch.randint(-8, 1, (T, r), generator=g).float() / 4).to(dtype)
        else:
            lx = torch.log_softmax(torch.randn(T, r, generator=g), -1).to(dtype)
            ly = torch.log_softmax(torch.randn(T, r, generator=g), -1).to(dtype)
        print(f"select case {case}: T={T} r={r} k={k} {dtype}", flush=True)
        want_s, want_i = oracle.router_select(lx, ly, r, k)
        s, i = hip.hip_omni_router_func(lx.to(device), ly.to(device), r, k)
        assert torch.equal(i.cpu(), want_i), (case, T, r, k, dtype)
        assert torch.equal(s.cpu().float(), want_s.float()), (case, T, r, k, dtype)


def test_schedule_random_shapes(device):
    rng = random.Random(99)
    hip = _ops()
    for case in range(40):
        N = rng.choice([1, 2, 7, 64, 100, 1000, 4096, 4097, 5000, 70000])
        T = rng.choice([1, 3, 64, 100, 1000, 5000])
        k = rng.choice([1, 2, 6, 16, 33])
        g = torch.Generator().manual_seed(case)
        lo, hi = (-2, N + 3) if rng.random() < 0.4 else (0, N)           # sometimes with ids outside [0, N)
        ids = torch.randint(lo, hi, (T, k), generator=g, dtype=torch.int32)
        if rng.random() < 0.3:
            ids[:, 0] = ids[0, 0]                                        # one hot expert
        print(f"schedule case {case}: T={T} k={k} N={N} ids in [{lo},{hi})", flush=True)
        got = hip.hip_omni_schedule_func(ids.to(device), N)
        flat = ids.reshape(-1).long()
        valid = (flat >= 0) & (flat < N)
        key = torch.where(valid, flat, torch.full_like(flat, N))
        order = torch.sort(key, stable=True).indices
        want_off = torch.zeros(N + 1, dtype=torch.int64)
        want_off[1:] = torch.cumsum(torch.bincount(flat[valid], minlength=N), 0)
        assert torch.equal(got.offsets.cpu().long(), want_off), case
        nv = int(valid.sum())
        assert torch.equal(got.sorted_pair_ids.cpu().long()[:nv], order[:nv]), case
        assert torch.equal(got.sorted_token_ids.cpu().long()[:nv], order[:nv] // k), case
        assert sorted(got.sorted_pair_ids.cpu().tolist()[nv:]) == sorted(order[nv:].tolist()), case


def test_expert_and_linear_random_shapes(device):
    rng = random.Random(7)
    hip = _ops()
    for case in range(40):
        dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        e = 4 if dtype == torch.float32 else 8
        H = e * rng.choice([1, 2, 5, 8, 16, 31, 32, 64, 65, 128])
        N = rng.choice([1, 3, 16, 100, 513])
        k = rng.choice([1, 2, 5, 8, 16])
        T = rng.choice([1, 4, 5, 63, 200, 4100])
        x, up, down, gates, ids = oracle.make_expert_inputs(case, T, H, N, min(k, N), dtype=dtype, w_std=0.1)
        print(f"expert case {case}: T={T} H={H} N={N} k={ids.size(1)} {dtype}", flush=True)
        want = oracle.expert_forward(x, up, down, gates, ids).float()
        d = [t.to(device) for t in (x, up, down, gates, ids)]
        scale = max(want.abs().max().item(), 1e-6)
        tol = (1e-2 if dtype != torch.float32 else 1e-5) * scale
        for algo in ("auto", "gather", "segment", "split"):
            try:
                got = hip.hip_omni_expert_func(*d, algo=algo).float().cpu()
            except ValueError:
                assert algo == "split"             # rows that do not cut into 8 power-of-two slices
                continue
            assert (got - want).abs().max().item() <= tol, (case, algo)
        # a linear layer of the same odd sizes: y = x W^T with W = up
        y = hip.hip_linear_func(d[0], d[1]).float().cpu()
        ref = x.double() @ up.double().t()
        ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -22}[dtype]
        assert ((y.double() - ref).abs() <= ulp * ref.abs() * 1.01 + 1e-4 * max(ref.abs().max().item(), 1e-6)).all(), case


def test_layer_random_shapes_fp32(device):
    """Whole layer in fp32 (where near-ties in the router are rare), train and eval, one and two streams."""
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    rng = random.Random(5)
    for case in range(12):
        H = 4 * rng.choice([4, 8, 9, 16, 33, 64])
        I = 4 * rng.choice([4, 8, 16, 17, 64])
        N = rng.choice([4, 9, 50, 64, 100, 257, 1024])
        r = int(N ** 0.5)
        k = 2 * rng.randint(1, max(1, min(8, r * r // 2)))
        T = rng.choice([1, 5, 64, 200, 777])
        training = rng.random() < 0.5 and T > 1         # batch statistics of one sample raise, as nn.BatchNorm1d does
        x, w = oracle.make_layer_inputs(100 + case, T, H, I, N, dtype=torch.float32, w_std=0.1)
        sd = {"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
              "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
              "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}
        print(f"layer case {case}: T={T} H={H} I={I} N={N} r={r} k={k} training={training}", flush=True)
        want, _, want_i = oracle.moe_forward(x, w, oracle.BNState.fresh(r), oracle.BNState.fresh(r), k, training)
        outs = []
        for overlap in (True, False):
            layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
            layer.load_state_dict(sd, strict=False)
            layer = layer.to(device).train(training)
            layer.overlap_branches, layer.overlap_min_work = overlap, 0
            with torch.no_grad():
                outs.append(layer(x.to(device)))
        assert torch.equal(outs[0], outs[1]), case
        scale = max(want.abs().max().item(), 1e-6)
        err = (outs[0].cpu() - want).abs().max().item()
        assert err <= 2e-4 * scale, (case, err, scale)
