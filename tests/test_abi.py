"""The C-ABI library loads without a GPU and exports exactly what include/omni_moe_hip.h declares.
No compute call is made here."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "omni_moe_hip.h")


def _declared():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"OMNI_API\s+[\w\s\*]+?\b(omni_\w+)\s*\(", text)))


def _lib():
    from omni_moe.ops.hip import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from omni_moe.ops.hip import build
        build.build_library()
    return _lib


def test_header_declares_the_path():
    names = _declared()
    for must in ("omni_router_select", "omni_router_fwd", "omni_schedule", "omni_expert_fwd", "omni_mlp_fwd"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = _lib().load()
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert lib.omni_abi_version() == 1
    assert b"ok" == lib.omni_error_string(0)
    assert b"NULL" in lib.omni_error_string(-1)


def test_binding_table_matches_header():
    lib = _lib()
    assert sorted(lib.SIGNATURES) == _declared()
    # argument counts of the ctypes table equal the header's parameter counts
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, args) in lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        params = [p for p in m.group(1).split(",") if p.strip() and p.strip() != "void"]
        assert len(params) == len(args), name


def test_no_extra_exports():
    lib = _lib()
    out = subprocess.run(["nm", "-D", "--defined-only", lib.LIB_PATH], capture_output=True, text=True).stdout
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T " in l and l.split()[-1].startswith("omni_"))
    assert exported == _declared()


def test_argument_errors_need_no_gpu():
    """Rejected arguments return before any HIP call, so these run on the CPU."""
    lib = _lib().load()
    p = ctypes.c_void_p(16)
    assert lib.omni_router_select(p, p, p, p, 4, 8, 3, 0, None) == -4          # odd k
    assert lib.omni_router_select(p, p, p, p, 4, 8, 66, 0, None) == -4         # k > r*r
    assert lib.omni_router_select(p, p, p, p, 4, 8, 4, 7, None) == -3          # dtype
    assert lib.omni_router_select(None, p, p, p, 4, 8, 4, 0, None) == -1       # NULL
    assert lib.omni_router_select(None, None, None, None, 0, 8, 4, 0, None) == 0   # no tokens: nothing to do
    assert lib.omni_expert_fwd(p, p, p, p, p, p, -1, 64, 16, 2, 0, 0, None, None) == -2
    assert lib.omni_expert_fwd(p, p, p, p, p, p, 4, 64, 16, 2, 9, 0, None, None) == -3
    assert lib.omni_schedule(p, p, p, p, 4, 2, 0, p, None) == -2
    assert lib.omni_schedule(p, p, p, p, 4, 2, 16, None, None) == -6
    assert lib.omni_mlp_fwd(p, p, p, p, None, p, 4, 64, 62, 0, p, None) == -2   # intermediate size not a multiple of 8
    # the whole layer: every stage's rule is checked before anything is enqueued
    moe = lambda H, I, N, r, k, dt=0: lib.omni_moe_fwd(*([p] * 15), 4, H, I, N, r, k, dt, 2, 0, 0.1, 1e-5, p, None, None, None, None)
    assert moe(64, 62, 16, 4, 2) == -2           # intermediate size
    assert moe(60, 64, 16, 4, 2) == -2           # hidden size
    assert moe(64, 64, 16, 4, 3) == -4           # odd k
    assert moe(64, 64, 16, 4, 18) == -4          # k > r*r
    assert moe(64, 64, 15, 4, 2) == -2           # r*r experts do not fit the tables
    assert moe(8200, 64, 16, 4, 2) == -5         # 16 400-byte rows: no cut into column blocks of 8 power-of-two slices
    assert moe(64, 64, 16, 4, 2, dt=5) == -3
    assert lib.omni_mlp_fwd(p, p, p, p, None, p, 4, 64, 64, 0, None, None) == -6 # no workspace
    assert lib.omni_schedule_workspace_bytes(4, 2, 100) >= 200
    # batch statistics of a single token: nn.BatchNorm1d raises in training (reference omni_moe.py:70-71), the library refuses
    assert lib.omni_moe_fwd(*([p] * 15), 1, 64, 64, 16, 4, 2, 0, 2, 1, 0.1, 1e-5, p, None, None, None, None) == -2
    assert lib.omni_router_fwd(*([p] * 9), 1, 0.1, 1e-5, p, p, None, 1, 64, 4, 2, 0, 2, p, None) == -2
    assert lib.omni_router_fwd(p, p, p, p, p, None, p, p, None, 1, -1.0, 1e-5, p, p, None, 4, 64, 4, 2, 0, 2, p, None) == -1   # cumulative average needs the counters
    # limits of the select kernels and of the schedule's multiply-shift division: refused before anything is enqueued
    assert lib.omni_router_fwd(*([p] * 9), 0, 0.1, 1e-5, p, p, None, 4, 64, 1025, 2, 2, 2, p, None) == -5      # r > 1024 with fp32 scores
    assert lib.omni_router_fwd(*([p] * 9), 0, 0.1, 1e-5, p, p, None, 4, 64, 1025, 66, 0, 2, p, None) == -5     # r > 1024 with k > 64
    assert lib.omni_router_select(p, p, p, p, 4, 1025, 2, 2, None) == -5
    assert lib.omni_router_select(p, p, p, p, 4, 16385, 2, 0, None) == -5                                       # r > 16384
    assert lib.omni_schedule(p, p, p, p, 1 << 20, 1024, 16, p, None) == -2                                      # 2^30 pairs
    import torch
    if not torch.cuda.is_available():
        assert lib.omni_init() >= 1000           # a HIP error (no device), not a crash


def test_schedule_token_id_division_is_exact():
    """The schedule writes sorted_token_ids = pair_id // top_k as (pair_id * ceil(2^s / top_k)) >> s with
    s = 30 + ceil(log2(top_k)) (schedule.hip); the entry points admit pair ids below 2^30.  Within that bound the
    multiply-shift must equal the integer division for every top_k, in 64-bit arithmetic.  Checked where it would
    break first: the last pair id before each multiple of top_k and the multiple itself, near the top of the range."""
    import numpy as np
    top = (1 << 30) - 1
    for k in list(range(1, 2100)) + [4095, 4096, 4097, 65535, 65537, (1 << 20) + 1, top]:
        s = 30
        while (1 << (s - 30)) < k:
            s += 1
        inv = ((1 << s) + k - 1) // k
        assert top * inv < 1 << 64                         # the product never wraps
        q = np.arange(max(top // k - 64, 0), top // k + 1, dtype=np.uint64)
        v = np.concatenate([q * np.uint64(k) + np.uint64(k - 1), q * np.uint64(k), np.arange(0, min(4 * k, 8192), dtype=np.uint64)])
        v = v[v <= top]
        assert np.array_equal((v * np.uint64(inv)) >> np.uint64(s), v // np.uint64(k)), k
    # a fixed shift of 40 is not enough beyond top_k = 1024 (and wraps for small top_k), which is why s follows top_k
    k, v = 1038, 1073741453
    assert (v * (((1 << 40) + k - 1) // k)) >> 40 != v // k


def test_ops_fail_loudly_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from omni_moe.ops import hip
    from omni_moe.ops.hip._lib import OmniHipError
    z = torch.zeros(4, 8)
    with pytest.raises(OmniHipError):
        hip.hip_omni_router_func(z, z, 8, 4)
    with pytest.raises(OmniHipError):
        hip.hip_omni_expert_func(torch.zeros(4, 8), torch.zeros(16, 8), torch.zeros(16, 8), torch.zeros(4, 2), torch.zeros(4, 2, dtype=torch.int32))


def test_reference_import_paths():
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    from omni_moe.ops.triton import triton_omni_expert_func, triton_omni_mlp_func, triton_omni_router_func  # noqa: F401
    layer = OmniMoE(OmniMoEConfig(64, 128, "silu", 256, 8))
    assert sorted(layer.state_dict()) == sorted([
        "gate_proj.weight", "up_proj.weight", "down_proj.weight", "router_gate_x.weight", "router_gate_y.weight",
        "router_norm_x.running_mean", "router_norm_x.running_var", "router_norm_x.num_batches_tracked",
        "router_norm_y.running_mean", "router_norm_y.running_var", "router_norm_y.num_batches_tracked",
        "up_embed.weight", "down_embed.weight"])
    assert layer.num_expert_sqrt == 16 and layer.up_embed.weight.shape == (256, 64)
    with pytest.raises(ValueError):
        OmniMoE(OmniMoEConfig(64, 128, "gelu", 256, 8))


def test_layer_is_a_plain_module_on_the_cpu(tmp_path):
    """Nothing on a layer stands in the way of copy.deepcopy, pickling or a state_dict round trip (the
    side stream and events of the two-stream forward live outside the module)."""
    import copy
    import torch
    from omni_moe.modules.omni_moe import OmniMoE, OmniMoEConfig
    layer = OmniMoE(OmniMoEConfig(64, 128, "silu", 256, 8))
    twin = copy.deepcopy(layer)
    assert all(torch.equal(a, b) for a, b in zip(layer.state_dict().values(), twin.state_dict().values()))
    path = str(tmp_path / "layer.pt")
    torch.save(layer, path)
    loaded = torch.load(path, weights_only=False)           # a file this test wrote itself
    assert sorted(loaded.state_dict()) == sorted(layer.state_dict())
    other = OmniMoE(OmniMoEConfig(64, 128, "silu", 256, 8))
    other.load_state_dict(layer.state_dict())
    assert torch.equal(other.up_embed.weight, layer.up_embed.weight)


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 (and C++), and a C program linked against the library
    runs its host-side entry points without a GPU."""
    inc = os.path.join(ROOT, "include")
    for cmd in (["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", HEADER],
                ["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", HEADER]):
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
    lib = _lib().LIB_PATH
    exe = str(tmp_path / "c_abi_client")
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", inc, os.path.join(ROOT, "tests", "c_abi_client.c"), lib,
                        "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath,/opt/rocm/lib", "-o", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "c abi ok" in r.stdout
