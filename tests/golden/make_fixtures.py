"""Writes tests/golden/omni_small.safetensors: small frozen input/output vectors of every operator on the path.

The reference ships no golden vectors and cannot be imported offline, so these come from the CPU oracle
(oracle/omni_oracle.py), whose functions are pinned by independent formulations in tests/test_oracle.py.  They
freeze the behaviour -- tie order, rounding points, BatchNorm buffer updates -- so that a later change to the oracle
or to a kernel shows up as a diff against committed numbers.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import torch
from safetensors.torch import save_file

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import omni_oracle as oracle  # noqa: E402


def build():
    out = {}
    g = torch.Generator().manual_seed(20240)
    # router select, bf16 scores on a coarse grid so that ties occur inside the halves and among the sums
    r, k, T = 8, 6, 12
    lx = (torch.randint(-6, 1, (T, r), generator=g).float() / 2).bfloat16()
    ly = (torch.randint(-6, 1, (T, r), generator=g).float() / 2).bfloat16()
    s, i = oracle.router_select(lx, ly, r, k)
    out.update({"router.lx": lx.float(), "router.ly": ly.float(), "router.scores": s.float(), "router.indices": i})
    # schedule
    ids = torch.randint(0, 8, (6, 4), generator=g, dtype=torch.int32)
    off, pairs = oracle.schedule(ids, 8)[:2]
    out.update({"schedule.indices": ids, "schedule.offsets": off.to(torch.int32), "schedule.sorted_pair_ids": pairs.to(torch.int32)})
    # experts, fp32
    x, up, down, gates, eid = oracle.make_expert_inputs(7, 5, 32, 16, 4, dtype=torch.float32, w_std=0.3)
    eid[0, 1] = eid[0, 0]                                         # a duplicate id adds twice
    out.update({"expert.x": x, "expert.up": up, "expert.down": down, "expert.gates": gates, "expert.indices": eid,
                "expert.y": oracle.expert_forward(x, up, down, gates, eid)})
    # the whole layer, fp32, train and eval from fresh buffers
    xl, w = oracle.make_layer_inputs(11, 8, 32, 64, 16, dtype=torch.float32, w_std=0.3)
    out["layer.x"] = xl
    for name in ("gate_proj", "up_proj", "down_proj", "router_gate_x", "router_gate_y", "up_embed", "down_embed"):
        out["layer." + name] = getattr(w, name)
    for mode, training in (("train", True), ("eval", False)):
        bx, by = oracle.BNState.fresh(4), oracle.BNState.fresh(4)
        y, gts, ix = oracle.moe_forward(xl, w, bx, by, 4, training)
        out.update({f"layer.{mode}.y": y, f"layer.{mode}.gates": gts, f"layer.{mode}.indices": ix.to(torch.int32),
                    f"layer.{mode}.running_mean_x": bx.running_mean.clone(), f"layer.{mode}.running_var_x": bx.running_var.clone()})
    return {key: v.contiguous() for key, v in out.items()}


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "omni_small.safetensors")
    save_file(build(), path)
    print(path, os.path.getsize(path), "bytes")
