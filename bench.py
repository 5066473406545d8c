"""Benchmark of the OmniMoE forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A step = one pass of the path over one batch of synthetic,
HBM-resident input.  Timing uses HIP events recorded on the stream the kernels run on
(torch's current stream; the library enqueues there).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "omni-moe_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published


def expert_alg_bytes(T, H, k, s=2):
    # per token: x row + k up rows + k down rows + y row, plus k ids (4 B) and k gates (s B)
    return T * ((2 * k + 2) * H * s + k * (4 + s))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)")

    import torch
    from omni_moe.ops import hip
    from oracle import omni_oracle as oracle          # checker + cpu_baseline leg only

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # BASELINE config 3: expert stage incl. the expert-centric sort
    T, H, N, k, seed = 16384, 1024, 4096, 16, 2
    x, up, down, gates, ids = oracle.make_expert_inputs(seed, T, H, N, k)
    dx, dup, ddown, dgates, dids = (t.to(dev) for t in (x, up, down, gates, ids))

    def step():
        hip.hip_omni_schedule_func(dids, N)
        return hip.hip_omni_expert_func(dx, dup, ddown, dgates, dids)

    for _ in range(a.warmup):
        y = step()
    torch.cuda.synchronize()
    # spot check against the oracle on a slice (checker, outside the timed region)
    want = oracle.expert_forward(x[:256], up, down, gates[:256], ids[:256])
    torch.testing.assert_close(y[:256].cpu().float(), want.float(), rtol=2e-2, atol=2e-2)

    # per-kernel duration of the expert kernel alone (events around each launch)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    s_all, e_all = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s_all.record()
    for s, e in evs:
        hip.hip_omni_schedule_func(dids, N)
        s.record()
        hip.hip_omni_expert_func(dx, dup, ddown, dgates, dids)
        e.record()
    e_all.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    total_ms = s_all.elapsed_time(e_all)
    ms_per_step = total_ms / a.steps
    kern_ms = sum(s.elapsed_time(e) for s, e in evs) / a.steps

    alg = expert_alg_bytes(T, H, k)
    achieved = alg / (kern_ms * 1e-3) / 1e9
    out = {
        "metric": "OmniMoE expert-stage fwd tokens/sec @h1024,N4096,k16 (1 GPU)",
        "value": T / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 3: schedule + fused expert, T=16384 H=1024 N=4096 k=16 bf16 seed 2"},
        "roofline": {"bound": "hbm", "kernel": "expert_gather_kernel", "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes": alg, "kernel_ms": kern_ms},
        "wall_s": wall,
    }
    if not a.no_cpu_baseline:
        # the oracle on the host cores, bounded sample of the same workload
        n = 2048
        torch.set_num_threads(min(16, os.cpu_count() or 1))
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 10.0:
            oracle.schedule(ids[:n], N)
            oracle.expert_forward(x[:n], up, down, gates[:n], ids[:n], compute_dtype=None)
            reps += 1
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": reps * n / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{reps} x first {n} tokens of the same workload, bf16 torch CPU ops (oracle restatement)"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
