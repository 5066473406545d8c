"""Benchmark of the OmniMoE forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A step = one forward of the OmniMoE layer over one batch of synthetic,
HBM-resident input: benchmark config 4, the README shape (1 x 4096 tokens, hidden 1024,
intermediate 4096, 4096 experts = 64 x 64 keys, top-16, bf16, train-mode BatchNorm).
All timing uses HIP events recorded on the stream the kernels run on (torch's current stream;
the library enqueues there).

  value      whole-layer tokens/s over the K timed steps
  roofline   the kernel that takes the largest share of a step (gate/up MFMA GEMM), timed per
             launch with events around its C-ABI call
  kernels    the same per-launch figures for every stage of the step, plus the fused expert
             kernel on benchmark config 3 (16384 tokens), the shape its bandwidth target is quoted on
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

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
# Fabric-side bytes per launch (FETCH_SIZE + WRITE_SIZE, each scaled by a plain copy of known size) from the
# rocprofv3 --pmc runs summarised in profiles/bench_layer_c4_hbm_counters.txt; counters cannot be read in-process.
TRAFFIC_BYTES = {"expert_c3": 183.2e6, "expert_c4": 57.8e6, "expert_gather_c3": 897.9e6, "gateup_c4": 134.7e6, "down_c4": 117.6e6}
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


EXPERT_NOTE = ("the 16 MiB up/down tables are served from the caches (each XCD's L2 holds the eighth of them its blocks use), "
               "so algorithmic bytes exceed fabric traffic and the fraction of HBM peak exceeds 1")


def expert_alg_bytes(T, H, k, s=2):
    """Gather model: per token the x row, k up rows, k down rows, the y row, k ids and k gates."""
    return T * ((2 * k + 2) * H * s + k * (4 + s))


def expert_bwd_alg_bytes(T, H, N, k, s=2):
    """Backward of the expert op.  Token pass: x, dy and dx rows, k up rows, k down rows, k ids, gates and dgates,
    k fp32 (ds, coef) pairs out.  Weight pass: per pair the x and dy rows, its two fp32 coefficients, pair id and token
    id; the dU and dV tables out.  Plus the schedule."""
    P = T * k
    token_pass = T * (2 * k + 3) * H * s + P * (4 + 2 * s + 8)
    weight_pass = P * (2 * H * s + 16) + 2 * N * H * s
    return token_pass + weight_pass + P * 14 + 8 * (N + 1)


def _events(torch, n):
    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


def time_call(torch, fn, reps, warmup=3):
    """Mean per-launch milliseconds of fn, HIP events around each call."""
    for _ in range(warmup):
        fn()
    ev = _events(torch, reps)
    torch.cuda.synchronize()
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return sum(s.elapsed_time(e) for s, e in ev) / reps


def hbm_entry(name, alg_bytes, ms, note=None, traffic=None):
    a = alg_bytes / (ms * 1e-3) / 1e9
    d = {"kernel": name, "bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
         "traffic": traffic, "algorithmic_bytes": alg_bytes, "kernel_ms": ms}
    if note:
        d["note"] = note
    return d


def mfma_entry(name, flops, ms, traffic=None):
    a = flops / (ms * 1e-3) / 1e12
    return {"kernel": name, "bound": "mfma", "achieved": a, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": a / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic, "algorithmic_flops": flops, "kernel_ms": ms}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel passes (profiling runs)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a plain 256 MiB device copy 3 times (known traffic, to scale HBM byte counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)")

    import torch
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    from omni_moe.ops import hip
    from oracle import omni_oracle as oracle          # checker + cpu_baseline leg only

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.set_grad_enabled(False)          # forward path: the module then issues its single fused library call

    # ---------------- benchmark config 4: README-shape full layer
    T, H, I, N, k, seed = 4096, 1024, 4096, 4096, 16, 3
    x, w = oracle.make_layer_inputs(seed, T, H, I, N)
    layer = OmniMoE(OmniMoEConfig(H, I, "silu", N, k))
    layer.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                           "router_gate_x.weight": w.router_gate_x, "router_gate_y.weight": w.router_gate_y,
                           "up_embed.weight": w.up_embed, "down_embed.weight": w.down_embed}, strict=False)
    layer = layer.to(device=dev, dtype=torch.bfloat16)          # module default: training mode (batch-stat BN)
    dx = x.to(dev)

    for _ in range(a.warmup):
        y = layer(dx)
    torch.cuda.synchronize()

    s_all, e_all = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    s_all.record()
    for _ in range(a.steps):
        y = layer(dx)
    e_all.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = s_all.elapsed_time(e_all) / a.steps

    out = {
        "metric": "OmniMoE fwd tokens/sec @h1024,N4096,k16 (1 GPU); expert kernel HBM GB/s %peak",
        "value": T / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[3] (benchmark config 4, the README shape): full OmniMoE layer forward, 1x4096 tokens, hidden 1024, intermediate 4096, "
                               "4096 experts (64x64), top-16, silu, train-mode BatchNorm, seed 3"},
        "wall_s_timed_region": wall,
    }

    # correctness spot check against the oracle (outside the timed region): eval mode on both
    # sides so that the repeated train-mode steps above do not matter
    layer.eval()
    sub = 256
    y_sub = layer(dx[:, :sub]).float().cpu()
    bx, by = oracle.BNState.fresh(layer.num_expert_sqrt), oracle.BNState.fresh(layer.num_expert_sqrt)
    bx.running_mean, bx.running_var = layer.router_norm_x.running_mean.float().cpu(), layer.router_norm_x.running_var.float().cpu()
    by.running_mean, by.running_var = layer.router_norm_y.running_mean.float().cpu(), layer.router_norm_y.running_var.float().cpu()
    want, _, _ = oracle.moe_forward(x[:, :sub], w, bx, by, k, training=False)
    torch.testing.assert_close(y_sub, want.float(), rtol=2e-2, atol=2e-2)
    layer.train()

    if a.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if not a.no_kernels:
        reps = max(10, min(a.steps, 50))
        xf = dx.view(-1, H)
        gates, ids = layer.route(xf)
        e_out = hip.hip_omni_expert_func(xf, layer.up_embed.weight, layer.down_embed.weight, gates, ids)
        h = hip.hip_swiglu_linear_func(xf, layer.gate_proj.weight, layer.up_proj.weight)
        ms_router = time_call(torch, lambda: layer.route(xf), reps)
        ms_expert = time_call(torch, lambda: hip.hip_omni_expert_func(xf, layer.up_embed.weight, layer.down_embed.weight, gates, ids), reps)
        ms_gateup = time_call(torch, lambda: hip.hip_swiglu_linear_func(xf, layer.gate_proj.weight, layer.up_proj.weight), reps)
        ms_down = time_call(torch, lambda: hip.hip_linear_func(h, layer.down_proj.weight, e_out), reps)
        r = layer.num_expert_sqrt
        kernels = [
            mfma_entry("gemm_nt_dma_kernel<swiglu> (gate/up projection + SwiGLU), c4", 4 * T * H * I, ms_gateup, TRAFFIC_BYTES["gateup_c4"]),
            mfma_entry("gemm_nt_dma_kernel<residual> (down projection + experts add), c4", 2 * T * H * I, ms_down, TRAFFIC_BYTES["down_c4"]),
            hbm_entry("expert op (split algorithm: expert_split_dots_kernel + expert_split_accumulate_kernel), c4", expert_alg_bytes(T, H, k),
                      ms_expert, EXPERT_NOTE, TRAFFIC_BYTES["expert_c4"]),
            {"kernel": "router stage (projection GEMM with BN statistics epilogue + BN finalize + select), c4", "kernel_ms": ms_router,
             "algorithmic_flops": 4 * T * H * r},
        ]
        # expert kernel at the shape its bandwidth target is quoted on (benchmark config 3)
        T3 = 16384
        x3, up3, down3, g3, i3 = (t.to(dev) for t in oracle.make_expert_inputs(2, T3, H, N, k))
        ms_e3 = time_call(torch, lambda: hip.hip_omni_expert_func(x3, up3, down3, g3, i3), reps)
        ms_g3 = time_call(torch, lambda: hip.hip_omni_expert_func(x3, up3, down3, g3, i3, algo="gather"), reps)
        ms_s3 = time_call(torch, lambda: hip.hip_omni_schedule_func(i3, N), reps)
        ms_seg3 = time_call(torch, lambda: hip.hip_omni_expert_func(x3, up3, down3, g3, i3, algo="segment"), reps)
        kernels.append(hbm_entry("expert op (split algorithm: expert_split_dots_kernel + expert_split_accumulate_kernel), c3 (T=16384)",
                                 expert_alg_bytes(T3, H, k), ms_e3, EXPERT_NOTE, TRAFFIC_BYTES["expert_c3"]))
        kernels.append(hbm_entry("expert op, gather algorithm (expert_gather_kernel), c3", expert_alg_bytes(T3, H, k), ms_g3,
                                 "for comparison: whole rows per wave, three quarters of them fetched over the fabric",
                                 TRAFFIC_BYTES["expert_gather_c3"]))
        kernels.append(hbm_entry("schedule (stable counting sort: count, scan x2, scatter, offsets), c3", T3 * k * 14 + 8 * (N + 1), ms_s3))
        kernels.append(hbm_entry("expert op, expert-centric 'segment' algorithm (schedule + scores pass + token pass), c3",
                                 expert_alg_bytes(T3, H, k), ms_seg3, "for comparison; same results as the gather algorithm"))
        out["roofline"] = max(kernels[:3], key=lambda d: d["kernel_ms"])
        out["roofline_expert"] = kernels[-4]
        # training path (not part of the forward metric): backward of the expert op at the same shape
        dy3 = x3 * 0.5
        ms_b3 = time_call(torch, lambda: hip.hip_omni_expert_bwd_func(dy3, x3, up3, down3, g3, i3), reps)
        kernels.append(hbm_entry("expert op backward (schedule + token pass + weight pass), c3", expert_bwd_alg_bytes(T3, H, N, k), ms_b3,
                                 "x, dy (32 MiB each) and the tables are cache-resident, so algorithmic bytes exceed HBM traffic"))
        out["kernels"] = kernels

    if not a.no_cpu_baseline:
        # the oracle (torch CPU restatement of the reference's PyTorch layer) on the host cores,
        # on the first 1024 tokens of the same workload, repeated for ~10 s
        n = 1024
        torch.set_num_threads(min(16, os.cpu_count() or 1))
        xs = x[:, :n].contiguous()
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0 or reps < 2:
            bx, by = oracle.BNState.fresh(layer.num_expert_sqrt), oracle.BNState.fresh(layer.num_expert_sqrt)
            oracle.moe_forward(xs, w, bx, by, k, training=True, expert_compute_dtype=None)
            reps += 1
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": reps * n / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{reps} forwards over the first {n} tokens of the same workload, "
                                         "bf16 torch CPU ops (oracle restatement of OmniMoE_Torch.forward)"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
