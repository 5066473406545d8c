"""Committed golden vectors (tests/golden/omni_small.safetensors, written by tests/golden/make_fixtures.py).
CPU: the oracle still reproduces them bit for bit.  GPU: the HIP operators reproduce them through the C ABI."""
import os

import pytest
import torch
from safetensors.torch import load_file

from oracle import omni_oracle as oracle

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "omni_small.safetensors")
WEIGHTS = ("gate_proj", "up_proj", "down_proj", "router_gate_x", "router_gate_y", "up_embed", "down_embed")


@pytest.fixture(scope="module")
def gold():
    return load_file(PATH)


def _weights(gold):
    return oracle.MoEWeights(**{n: gold["layer." + n] for n in WEIGHTS})


def test_oracle_reproduces_the_fixture(gold):
    s, i = oracle.router_select(gold["router.lx"].bfloat16(), gold["router.ly"].bfloat16(), 8, 6)
    assert torch.equal(s.float(), gold["router.scores"]) and torch.equal(i, gold["router.indices"])
    off, pairs, _ = oracle.schedule(gold["schedule.indices"], 8)
    assert torch.equal(off, gold["schedule.offsets"]) and torch.equal(pairs, gold["schedule.sorted_pair_ids"])
    y = oracle.expert_forward(*(gold["expert." + n] for n in ("x", "up", "down", "gates", "indices")))
    assert torch.equal(y, gold["expert.y"])
    for mode, training in (("train", True), ("eval", False)):
        bx, by = oracle.BNState.fresh(4), oracle.BNState.fresh(4)
        y, g, ix = oracle.moe_forward(gold["layer.x"], _weights(gold), bx, by, 4, training)
        assert torch.equal(y, gold[f"layer.{mode}.y"]) and torch.equal(ix.to(torch.int32), gold[f"layer.{mode}.indices"])
        assert torch.equal(bx.running_mean, gold[f"layer.{mode}.running_mean_x"])
        assert torch.equal(bx.running_var, gold[f"layer.{mode}.running_var_x"])


def test_fixture_is_self_consistent(gold):
    """What the numbers must satisfy whoever computed them: every id reproduces its score, scores descend, ties go to
    the lower candidate; offsets are the prefix sums of the id histogram; the duplicate id in the expert case adds."""
    lx, ly, s, i = gold["router.lx"], gold["router.ly"], gold["router.scores"], gold["router.indices"].long()
    assert torch.equal((lx.gather(1, i // 8) + ly.gather(1, i % 8)).bfloat16().float(), s)
    assert (s[:, :-1] >= s[:, 1:]).all()
    full = (lx.unsqueeze(2) + ly.unsqueeze(1)).reshape(lx.size(0), 64).bfloat16().float()
    assert torch.equal(full.topk(6, dim=1).values, s)                  # the values of a top-k do not depend on tie order
    ids = gold["schedule.indices"].long().flatten()
    assert torch.equal(gold["schedule.offsets"].long()[1:], torch.bincount(ids, minlength=8).cumsum(0))
    assert torch.equal(ids[gold["schedule.sorted_pair_ids"].long()], ids.sort().values)
    x, up, down, gates, eid = (gold["expert." + n] for n in ("x", "up", "down", "gates", "indices"))
    t0 = sum(torch.nn.functional.silu(x[0] @ up[e]) * gates[0, j] * down[e] for j, e in enumerate(eid[0].tolist()))
    torch.testing.assert_close(gold["expert.y"][0], t0, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_hip_operators_reproduce_the_fixture(gold, device):
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    from omni_moe.ops import hip
    d = lambda t: t.to(device)
    s, i = hip.hip_omni_router_func(d(gold["router.lx"].bfloat16()), d(gold["router.ly"].bfloat16()), 8, 6)
    assert torch.equal(s.float().cpu(), gold["router.scores"]) and torch.equal(i.cpu(), gold["router.indices"])
    sched = hip.hip_omni_schedule_func(d(gold["schedule.indices"]), 8)
    assert torch.equal(sched.offsets.cpu(), gold["schedule.offsets"])
    assert torch.equal(sched.sorted_pair_ids.cpu(), gold["schedule.sorted_pair_ids"])
    y = hip.hip_omni_expert_func(*(d(gold["expert." + n]) for n in ("x", "up", "down", "gates", "indices")))
    torch.testing.assert_close(y.cpu(), gold["expert.y"], rtol=1e-5, atol=1e-6)
    for mode, training in (("train", True), ("eval", False)):
        layer = OmniMoE(OmniMoEConfig(32, 64, "silu", 16, 4))
        layer.load_state_dict({n + ".weight": gold["layer." + n] for n in WEIGHTS}, strict=False)
        layer = layer.to(device).train(training)
        with torch.no_grad():
            got = layer(d(gold["layer.x"]))
        torch.testing.assert_close(got.cpu(), gold[f"layer.{mode}.y"], rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(layer.router_norm_x.running_mean.cpu(), gold[f"layer.{mode}.running_mean_x"], rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(layer.router_norm_x.running_var.cpu(), gold[f"layer.{mode}.running_var_x"], rtol=1e-5, atol=1e-6)
