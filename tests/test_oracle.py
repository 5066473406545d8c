"""Pins the CPU oracle (oracle/omni_oracle.py) against independent formulations.

The reference ships no golden vectors (its tests only time kernels and print
mismatches), so each oracle function is checked against a torch *library* routine of the
same mathematics, a brute-force loop on tiny inputs, or an invariant -- never against a
retyped copy of its own formula.  Runs on the CPU.
"""
import itertools
import math

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import omni_oracle as oracle


# ----------------------------------------------------------------- batch_norm / log_softmax
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("training", [True, False])
def test_batch_norm_matches_torch_module(dtype, training):
    g = torch.Generator().manual_seed(0)
    T, r = 257, 48
    z = (torch.randn(T, r, generator=g) * 3 + torch.randn(r, generator=g)).to(dtype)
    bn = nn.BatchNorm1d(r, affine=False)
    bn.running_mean.copy_(torch.randn(r, generator=g) * 0.2)
    bn.running_var.copy_(torch.rand(r, generator=g) + 0.5)
    rm, rv = bn.running_mean.clone(), bn.running_var.clone()
    bn.train(training)
    want = bn(z.float())                                   # library routine, fp32
    got = oracle.batch_norm(z, rm, rv, training)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.float(), want, **tol)
    torch.testing.assert_close(rm, bn.running_mean, rtol=1e-5, atol=1e-6)     # momentum update, unbiased var
    torch.testing.assert_close(rv, bn.running_var, rtol=1e-5, atol=1e-6)
    if training:                                           # invariants of batch statistics
        n = oracle.batch_norm(z.float(), rm.clone(), rv.clone(), True, update=False)
        assert n.mean(0).abs().max() < 1e-5
        torch.testing.assert_close(n.var(0, unbiased=False), torch.ones(r), rtol=1e-3, atol=1e-3)


def test_batch_norm_cumulative_average_and_single_sample():
    """momentum=None: the module averages the batch statistics cumulatively (factor 1 / num_batches_tracked); a single
    sample in training raises, as nn.BatchNorm1d does."""
    g = torch.Generator().manual_seed(3)
    r = 24
    bn = nn.BatchNorm1d(r, affine=False, momentum=None).train()
    st = oracle.BNState.fresh(r)
    for step in range(4):
        z = torch.randn(50 + step, r, generator=g) * (1 + step) + step
        want = bn(z)
        got = oracle.batch_norm(z, st.running_mean, st.running_var, True, momentum=None, num_batches_tracked=st.num_batches_tracked)
        st.num_batches_tracked += 1
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(st.running_mean, bn.running_mean, rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(st.running_var, bn.running_var, rtol=1e-5, atol=1e-6)
    assert int(st.num_batches_tracked) == int(bn.num_batches_tracked) == 4
    with pytest.raises(ValueError):
        oracle.batch_norm(torch.randn(1, r), st.running_mean, st.running_var, True)
    with pytest.raises(ValueError):
        bn(torch.randn(1, r))
    oracle.batch_norm(torch.randn(1, r), st.running_mean, st.running_var, False)      # eval takes one sample


def test_batch_norm_bf16_matches_functional():
    g = torch.Generator().manual_seed(1)
    z = torch.randn(512, 64, generator=g).bfloat16()
    got = oracle.batch_norm(z, torch.zeros(64), torch.ones(64), True, update=False)
    # fp32 statistics and arithmetic, one rounding at the end (what torch's GPU batch-norm kernels
    # do for 16-bit inputs): the library routine on the upcast input, rounded once
    want = F.batch_norm(z.float(), None, None, training=True).bfloat16()
    assert (got == want).float().mean() > 0.999
    assert (got.float() - want.float()).abs().max() <= 2 ** -6          # <= 1 ulp at |v| < 4
    # torch's CPU bf16 kernel folds mean and invstd into a scale and shift first; it stays within 2 ulp
    cpu16 = F.batch_norm(z, None, None, training=True)
    assert (got.float() - cpu16.float()).abs().max() <= 2 ** -5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_log_softmax_matches_torch(dtype):
    g = torch.Generator().manual_seed(2)
    l = (torch.randn(300, 64, generator=g) * 4).to(dtype)
    got, want = oracle.log_softmax(l), torch.log_softmax(l, -1)
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
        assert torch.logsumexp(got, -1).abs().max() < 1e-5
    else:
        # fp32 inside, one rounding (torch's GPU kernels): the library routine on the upcast input
        w32 = torch.log_softmax(l.float(), -1).to(dtype)
        assert (got == w32).float().mean() > 0.999
        # torch's CPU 16-bit kernel rounds an intermediate as well: within one ulp of it
        assert (got == want).float().mean() > 0.9
        assert (got.float() - want.float()).abs().max() <= (2 ** -3 if dtype == torch.bfloat16 else 2 ** -6)


# ----------------------------------------------------------------- router_select
def _brute_force(lx, ly, r, k):
    """Top-k over the FULL r*r outer sum (what the reference's own test does with topk(num_keys),
    tests/test_router.py:14-21), formed in the input dtype."""
    full = (lx.unsqueeze(-1) + ly.unsqueeze(-2)).reshape(lx.size(0), r * r)
    return torch.topk(full.float(), k, dim=-1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r,k", [(8, 4), (16, 16), (32, 8), (64, 16), (6, 36), (100, 10)])
def test_router_select_against_brute_force(r, k, dtype):
    g = torch.Generator().manual_seed(r * 100 + k)
    T = 200
    lx = torch.log_softmax(torch.randn(T, r, generator=g), -1).to(dtype)
    ly = torch.log_softmax(torch.randn(T, r, generator=g), -1).to(dtype)
    s, i = oracle.router_select(lx, ly, r, k)
    assert s.dtype == dtype and i.dtype == torch.int32 and s.shape == (T, k)
    bs, bi = _brute_force(lx, ly, r, k)
    # (iii) the selected VALUES do not depend on how ties break: equal to topk bit for bit
    assert torch.equal(s.float(), bs)
    # (iv) every id reproduces its score
    ix, iy = (i // r).long(), (i % r).long()
    assert torch.equal((lx.gather(1, ix) + ly.gather(1, iy)).float(), s.float())
    # ids distinct inside a token, in range
    assert (i >= 0).all() and (i < r * r).all()
    assert all(len(set(row.tolist())) == k for row in i)
    # (v) where a token's k+1 best sums are strictly distinct the ids are forced
    bs1 = torch.topk((lx.unsqueeze(-1) + ly.unsqueeze(-2)).reshape(T, r * r).float(), min(k + 1, r * r), dim=-1).values
    strict = (bs1[:, :-1] > bs1[:, 1:]).all(-1) if k < r * r else (bs[:, :-1] > bs[:, 1:]).all(-1)
    assert strict.any() or dtype != torch.float32     # 16-bit sums tie often; fp32 ones never do
    assert torch.equal(i[strict].long(), bi[strict])


def test_router_select_tie_rules():
    r, k = 4, 4
    # all equal: per half the lower key index ranks first, candidates in position order a*k'+b
    z = torch.zeros(1, r)
    s, i = oracle.router_select(z, z, r, k)
    assert i.tolist() == [[0, 1, 2, 3]] and s.tolist() == [[0.0] * 4]
    # x = [1,1,0,0], y = [1,0,1,0]: sums 2 (0,0),(1,0)... enumerate by hand
    lx = torch.tensor([[1.0, 1.0, 0.0, 0.0]])
    ly = torch.tensor([[1.0, 0.0, 1.0, 0.0]])
    # sorted x keys: [0,1,2,3] scores [1,1,0,0]; sorted y keys: [0,2,1,3] scores [1,1,0,0]
    # candidates in position order: (a=0,b=0)->2 id 0*4+0; (0,1)->2 id 0*4+2; (0,2)->1 ...; (1,0)->2 id 4; (1,1)->2 id 6
    s, i = oracle.router_select(lx, ly, r, k)
    assert s.tolist() == [[2.0, 2.0, 2.0, 2.0]]
    assert i.tolist() == [[0, 2, 4, 6]]
    # the reference kernel's rule restated as its literal loop: k rounds of (max, first argmax, mask)
    g = torch.Generator().manual_seed(3)
    lx = (torch.randn(64, 8, generator=g) * 2).round() / 2
    ly = (torch.randn(64, 8, generator=g) * 2).round() / 2
    s, i = oracle.router_select(lx, ly, 8, 6)
    for t in range(64):
        sx, ixs = torch.sort(lx[t], descending=True, stable=True)
        sy, iys = torch.sort(ly[t], descending=True, stable=True)
        kp = 6
        cand = (sx[:kp, None] + sy[None, :kp]).reshape(-1).clone()
        for j in range(6):
            p = int(torch.argmax(cand))                     # first maximal position
            assert i[t, j].item() == ixs[p // kp].item() * 8 + iys[p % kp].item()
            assert s[t, j].item() == cand[p].item()
            cand[p] = -math.inf


def test_router_select_contract():
    z = torch.zeros(2, 8)
    for bad_k in (3, 66, 130):
        with pytest.raises(AssertionError):
            oracle.router_select(z, z, 8, bad_k)
    s, i = oracle.router_select(z, z, 8, 0)
    assert s.shape == (2, 0)


# ----------------------------------------------------------------- schedule
def test_schedule_against_loop_and_library():
    g = torch.Generator().manual_seed(4)
    T, k, N = 37, 6, 20
    ids = torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)
    off, pairs, tok = oracle.schedule(ids, N)
    buckets = [[] for _ in range(N)]
    for t in range(T):
        for j in range(k):
            buckets[ids[t, j].item()].append(t * k + j)
    flat = list(itertools.chain.from_iterable(buckets))
    assert pairs.tolist() == flat                                       # stable: ascending pair id per expert
    assert off.tolist() == [0] + list(itertools.accumulate(len(b) for b in buckets))
    assert tok.tolist() == [p // k for p in flat]
    assert torch.equal(off[1:] - off[:-1], torch.bincount(ids.flatten().long(), minlength=N).int())
    # same segments as the reference's compact form (unique_consecutive over the sorted ids)
    sorted_ids = ids.flatten()[pairs.long()]
    uniq, counts = torch.unique_consecutive(sorted_ids, return_counts=True)
    assert torch.equal(counts.int(), (off[1:] - off[:-1])[uniq.long()])


# ----------------------------------------------------------------- expert / mlp / layer
def test_expert_forward_against_loop_and_invariants():
    g = torch.Generator().manual_seed(5)
    T, H, N, k = 9, 16, 12, 4
    x, up, down = torch.randn(T, H, generator=g), torch.randn(N, H, generator=g), torch.randn(N, H, generator=g)
    gates = torch.randn(T, k, generator=g)
    ids = torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)     # duplicates allowed
    got = oracle.expert_forward(x, up, down, gates, ids)
    want = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = ids[t, j].item()
            s = float(torch.dot(x[t].double(), up[e].double()))
            want[t] += (s / (1 + math.exp(-s))) * float(gates[t, j]) * down[e].double()
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    # the reference's own restatement (tests/test_expert.py:8-25), from library ops
    ref = torch.matmul((F.silu(torch.matmul(up[ids.long()], x.unsqueeze(-1)).view(T, -1)) * gates).unsqueeze(-2),
                       down[ids.long()]).squeeze(-2)
    torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-5)
    # linear in the gates; invariant under a permutation of the k slots; duplicates add
    torch.testing.assert_close(oracle.expert_forward(x, up, down, 3 * gates, ids), 3 * got, rtol=1e-5, atol=1e-5)
    perm = torch.tensor([2, 0, 3, 1])
    torch.testing.assert_close(oracle.expert_forward(x, up, down, gates[:, perm], ids[:, perm]), got, rtol=1e-5, atol=1e-5)
    dup_ids, dup_g = torch.full((T, 2), 5, dtype=torch.int32), torch.ones(T, 2)
    one = oracle.expert_forward(x, up, down, torch.ones(T, 1), torch.full((T, 1), 5, dtype=torch.int32))
    torch.testing.assert_close(oracle.expert_forward(x, up, down, dup_g, dup_ids), 2 * one, rtol=1e-5, atol=1e-5)
    # chunking is exact
    torch.testing.assert_close(oracle.expert_forward(x, up, down, gates, ids, chunk=2), got, rtol=0, atol=0)


def test_mlp_forward_against_float64():
    g = torch.Generator().manual_seed(6)
    T, H, I = 11, 24, 40
    x, wg, wu, wd = (torch.randn(*s, generator=g) for s in ((T, H), (I, H), (I, H), (H, I)))
    want = (F.silu(x.double() @ wg.double().t()) * (x.double() @ wu.double().t())) @ wd.double().t()
    torch.testing.assert_close(oracle.mlp_forward(x, wg, wu, wd).double(), want, rtol=1e-4, atol=1e-4)
    # bf16: the rounding points are those of the reference's in-test restatement (tests/test_mlp.py:8-21)
    xb, gb, ub, db = (t.bfloat16() for t in (x, wg, wu, wd))
    ref = torch.matmul((F.silu(torch.matmul(xb, gb.t()).float()) * torch.matmul(xb, ub.t()).float()).bfloat16(), db.t())
    assert torch.equal(oracle.mlp_forward(xb, gb, ub, db), ref)


class _TorchLayer(nn.Module):
    """The layer assembled from torch.nn parts by the reference's definition
    (omni_moe/modules/omni_moe.py:109-194), written with library calls only: independent of
    the oracle's helper functions (F.batch_norm via nn.BatchNorm1d, torch.topk, nn.Embedding)."""

    def __init__(self, H, I, N, k):
        super().__init__()
        r = math.floor(math.sqrt(N))
        self.r, self.k = r, k
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(H, I, bias=False), nn.Linear(H, I, bias=False), nn.Linear(I, H, bias=False)
        self.router_gate_x, self.router_gate_y = nn.Linear(H, r, bias=False), nn.Linear(H, r, bias=False)
        self.router_norm_x, self.router_norm_y = nn.BatchNorm1d(r, affine=False), nn.BatchNorm1d(r, affine=False)
        self.up_embed, self.down_embed = nn.Embedding(N, H), nn.Embedding(N, H)

    def forward(self, h):
        B, S, H = h.shape
        x = h.view(-1, H)
        px = F.log_softmax(self.router_norm_x(self.router_gate_x(x)), -1)
        py = F.log_softmax(self.router_norm_y(self.router_gate_y(x)), -1)
        kp = min(self.r, self.k)
        sx, ix = px.topk(kp, -1)
        sy, iy = py.topk(kp, -1)
        alls = (sx.unsqueeze(-1) + sy.unsqueeze(-2)).flatten(-2)
        alli = (ix.unsqueeze(-1) * self.r + iy.unsqueeze(-2)).flatten(-2)
        s, pos = alls.topk(self.k, -1)
        idx = alli.gather(-1, pos)
        w = torch.exp(s)
        ew = torch.matmul(self.up_embed(idx), x.view(B * S, -1, 1)).view(B * S, -1)
        ew = F.silu(ew) * w
        es = torch.matmul(ew.view(B * S, 1, -1), self.down_embed(idx)).view(B, S, -1)
        return self.down_proj(F.silu(self.gate_proj(h)) * self.up_proj(h)) + es, idx


@pytest.mark.parametrize("training", [True, False])
def test_moe_forward_matches_torch_layer_fp32(training):
    """benchmark config 1 (the reference's CPU-runnable case) at reduced size, fp32."""
    T, H, I, N, k = 128, 64, 256, 256, 8
    x, w = oracle.make_layer_inputs(0, T, H, I, N, dtype=torch.float32)
    layer = _TorchLayer(H, I, N, k)
    with torch.no_grad():
        for name in ("gate_proj", "up_proj", "down_proj", "router_gate_x", "router_gate_y", "up_embed", "down_embed"):
            getattr(layer, name).weight.copy_(getattr(w, name))
    layer.train(training)
    r = layer.r
    bx, by = oracle.BNState.fresh(r), oracle.BNState.fresh(r)
    with torch.no_grad():
        want, want_idx = layer(x)
    got, gates, ids = oracle.moe_forward(x, w, bx, by, k, training)
    # fp32 random scores: ties have probability ~0, so ids are forced
    assert torch.equal(ids.long().sort(-1).values, want_idx.sort(-1).values)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    if training:
        torch.testing.assert_close(bx.running_mean, layer.router_norm_x.running_mean, rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(by.running_var, layer.router_norm_y.running_var, rtol=1e-5, atol=1e-6)
        assert bx.num_batches_tracked.item() == 1


def test_moe_forward_config1_full_size_runs():
    """benchmark config 1 at full size (T=512, H=256, I=1024, N=1024, k=8, fp32, seed 0)."""
    x, w = oracle.make_layer_inputs(0, 512, 256, 1024, 1024, dtype=torch.float32)
    bx, by = oracle.BNState.fresh(32), oracle.BNState.fresh(32)
    y, gates, ids = oracle.moe_forward(x, w, bx, by, 8, training=True)
    assert y.shape == (1, 512, 256) and ids.shape == (512, 8) and torch.isfinite(y).all()
    assert (gates > 0).all() and (gates.sum(-1) < 1).all()          # gates are joint probabilities, not renormalised
    assert (gates[:, :-1] >= gates[:, 1:]).all()
