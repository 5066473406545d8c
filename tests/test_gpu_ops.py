"""GPU parity of the HIP operators against the CPU oracle (same seeded inputs).

Every call goes through the C ABI (ctypes -> libomni_moe_hip.so).  Bars:
index / integer results bit-exact; scores bit-exact (they are sums of two inputs
rounded once); floating outputs within rtol=atol=2e-2 for 16-bit storage and
1e-4 / 1e-5 for fp32 storage.
"""
import pytest
import torch

from oracle import omni_oracle as oracle

pytestmark = pytest.mark.gpu


def _ops():
    from omni_moe.ops import hip
    return hip


# ---------------------------------------------------------------- router select
ROUTER_CASES = [
    # (T, r, k, dtype, kind)  -- first six are the reference benchmark grid (tests/test_router.py:103-110)
    (1024, 64, 16, torch.bfloat16, "randn"),
    (1024, 64, 32, torch.bfloat16, "randn"),
    (1024, 128, 16, torch.bfloat16, "randn"),
    (1024, 128, 32, torch.bfloat16, "randn"),
    (1024, 256, 16, torch.bfloat16, "randn"),
    (1024, 256, 32, torch.bfloat16, "randn"),
    (4096, 64, 16, torch.bfloat16, "logprob"),     # benchmark config 2 shape
    (2048, 512, 32, torch.bfloat16, "logprob"),    # benchmark config 5 shape (token subset)
    (512, 32, 8, torch.float32, "logprob"),        # benchmark config 1 shape
    (333, 64, 16, torch.float16, "randn"),
    (257, 100, 10, torch.bfloat16, "randn"),       # r not a multiple of 64
    (64, 4, 16, torch.bfloat16, "randn"),          # k = r*r: every expert selected, k' = r
    (64, 8, 32, torch.float32, "randn"),           # k > r
    (100, 128, 128, torch.bfloat16, "randn"),      # largest k the contract allows
    (100, 1024, 64, torch.bfloat16, "randn"),      # largest r the kernels hold in registers
    (70, 1025, 2, torch.bfloat16, "randn"),        # beyond: the row is walked in chunks of 512 keys (16-bit scores, k <= 64)
    (50, 1500, 16, torch.bfloat16, "logprob"),
    (40, 2048, 64, torch.float16, "randn"),
    (30, 4096, 32, torch.bfloat16, "ties"),
    (9, 16384, 8, torch.bfloat16, "randn"),
    (512, 64, 16, torch.bfloat16, "ties"),         # heavy ties: scores on a coarse grid
    (512, 64, 16, torch.float32, "allequal"),      # all scores equal: pure tie-break
    (1, 64, 2, torch.bfloat16, "randn"),
]


def _router_inputs(T, r, dtype, kind, seed):
    g = torch.Generator().manual_seed(seed)
    a, b = torch.randn(T, r, generator=g), torch.randn(T, r, generator=g)
    if kind == "logprob":
        a, b = torch.log_softmax(a, -1), torch.log_softmax(b, -1)
    elif kind == "ties":
        a, b = (a * 2).round() / 2, (b * 2).round() / 2
    elif kind == "allequal":
        a, b = torch.zeros(T, r), torch.zeros(T, r)
    return a.to(dtype), b.to(dtype)


@pytest.mark.parametrize("case", ROUTER_CASES, ids=lambda c: f"T{c[0]}-r{c[1]}-k{c[2]}-{str(c[3]).split('.')[-1]}-{c[4]}")
def test_router_select_bit_exact(case, device):
    T, r, k, dtype, kind = case
    lx, ly = _router_inputs(T, r, dtype, kind, seed=T + r + k)
    print(f"router_select T={T} r={r} k={k} {dtype} {kind}", flush=True)
    want_s, want_i = oracle.router_select(lx, ly, r, k)
    got_s, got_i = _ops().hip_omni_router_func(lx.to(device), ly.to(device), r, k)
    torch.cuda.synchronize()
    assert got_s.dtype == dtype and got_i.dtype == torch.int32 and got_s.shape == (T, k)
    assert torch.equal(got_s.cpu().float(), want_s.float())
    assert torch.equal(got_i.cpu(), want_i)


def test_router_select_contract(device):
    hip = _ops()
    lx = torch.zeros(4, 8, device=device)
    with pytest.raises(AssertionError):
        hip.hip_omni_router_func(lx, lx, 8, 3)          # odd k
    with pytest.raises(AssertionError):
        hip.hip_omni_router_func(lx, lx, 8, 66)         # k > r*r
    with pytest.raises(AssertionError):
        hip.hip_omni_router_func(lx, lx[:2], 8, 4)      # token counts differ
    s, i = hip.hip_omni_router_func(lx, lx, 8, 0)       # k = 0 is legal: empty result
    assert s.shape == (4, 0) and i.shape == (4, 0)
    s, i = hip.hip_omni_router_func(lx[:0], lx[:0], 8, 4)
    assert s.shape == (0, 4)
    # non-contiguous input is copied, as the reference does
    wide = torch.randn(16, 128, device=device)
    s1, i1 = hip.hip_omni_router_func(wide[:, ::2], wide[:, 1::2], 64, 16)
    s2, i2 = hip.hip_omni_router_func(wide[:, ::2].contiguous(), wide[:, 1::2].contiguous(), 64, 16)
    assert torch.equal(s1, s2) and torch.equal(i1, i2)


# ---------------------------------------------------------------- schedule
SCHED_CASES = [(512, 8, 1024, "uniform"), (4096, 16, 4096, "uniform"), (16384, 16, 4096, "uniform"),
               (4096, 32, 262144, "zipf"), (1000, 6, 5000, "zipf"), (3, 2, 7, "uniform"), (2048, 16, 64, "hot"),
               (32768, 32, 262144, "zipf"), (777, 10, 1048576, "uniform"), (100, 4, 1, "hot"), (5000, 8, 4097, "uniform"),
               # more than 256 tiles of 8192 pairs (tiles grow), and tiles at their 16-bit limit with every pair in one bin
               (150000, 16, 4096, "uniform"), (1100000, 16, 4096, "hot")]


def _sched_ids(T, k, N, kind, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "uniform":
        return torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)
    if kind == "hot":
        return torch.zeros(T, k, dtype=torch.int32)
    w = 1.0 / torch.arange(1, N + 1, dtype=torch.float64) ** 1.1
    return torch.multinomial(w, T * k, replacement=True, generator=g).reshape(T, k).to(torch.int32)


@pytest.mark.parametrize("case", SCHED_CASES, ids=lambda c: f"T{c[0]}-k{c[1]}-N{c[2]}-{c[3]}")
def test_schedule_matches_oracle(case, device):
    T, k, N, kind = case
    ids = _sched_ids(T, k, N, kind, seed=T + k)
    print(f"schedule T={T} k={k} N={N} {kind}", flush=True)
    want_off, want_pairs, want_tok = oracle.schedule(ids, N)
    got = _ops().hip_omni_schedule_func(ids.to(device), N)
    torch.cuda.synchronize()
    off, pairs, tok = got.offsets.cpu(), got.sorted_pair_ids.cpu(), got.sorted_token_ids.cpu()
    assert torch.equal(off, want_off)
    assert torch.equal(pairs, want_pairs)                  # stable: bit-exact against torch.sort(stable=True)
    assert torch.equal(tok, (pairs // k).to(torch.int32))
    again = _ops().hip_omni_schedule_func(ids.to(device), N)
    assert torch.equal(again.sorted_pair_ids.cpu(), pairs)  # and identical from run to run


# ---------------------------------------------------------------- expert
EXPERT_CASES = [
    # (T, H, N, k, dtype, kind)
    (1024, 1024, 1024, 32, torch.bfloat16, "ref"),      # reference benchmark grid (tests/test_expert.py:181-187)
    (1024, 1024, 4096, 32, torch.bfloat16, "ref"),
    (1024, 1024, 16384, 32, torch.bfloat16, "ref"),     #   ... its two larger tables: 64 MiB and 256 MiB
    (1024, 1024, 65536, 32, torch.bfloat16, "ref"),
    (4096, 1024, 16384, 16, torch.bfloat16, "ref"),     # 65536 pairs, 64 MiB of tables: AUTO takes the hidden-split algorithm
    (2048, 1024, 4096, 16, torch.bfloat16, "baseline"), # benchmark config 3 shape (token subset)
    (512, 256, 1024, 8, torch.float32, "baseline"),     # benchmark config 1 shape
    (256, 2048, 8192, 32, torch.bfloat16, "baseline"),  # benchmark config 5 row length
    (130, 1024, 512, 6, torch.float16, "ref"),
    (77, 520, 300, 10, torch.bfloat16, "ref"),          # H not a multiple of 512
    (64, 4096, 256, 4, torch.bfloat16, "ref"),
    (5, 64, 16, 2, torch.float32, "ref"),
]


def _expert_inputs(T, H, N, k, dtype, kind, seed):
    if kind == "baseline":
        return oracle.make_expert_inputs(seed, T, H, N, k, dtype)
    # the reference's benchmark distribution (tests/test_expert.py:83-98): negative gates
    # occur, ids are drawn with replacement so a token can repeat an expert
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, H, generator=g) * 0.5).to(dtype)
    up = (torch.randn(N, H, generator=g) * 0.1).to(dtype)
    down = (torch.randn(N, H, generator=g) * 0.1).to(dtype)
    gates = (torch.randn(T, k, generator=g) * 0.1).to(dtype)
    ids = torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)
    return x, up, down, gates, ids


def _tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype != torch.float32 else dict(rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("case", EXPERT_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-N{c[2]}-k{c[3]}-{str(c[4]).split('.')[-1]}-{c[5]}")
def test_expert_matches_oracle(case, device):
    T, H, N, k, dtype, kind = case
    x, up, down, gates, ids = _expert_inputs(T, H, N, k, dtype, kind, seed=T + H)
    print(f"expert T={T} H={H} N={N} k={k} {dtype} {kind}", flush=True)
    want = oracle.expert_forward(x, up, down, gates, ids)                 # fp32 sums, one rounding
    got = _ops().hip_omni_expert_func(*(t.to(device) for t in (x, up, down, gates, ids)))
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == (T, H)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))
    # tighter, scale-aware check: the two differ only by fp32 summation order + one rounding
    err = (got.cpu().float() - want.float()).abs().max().item()
    scale = want.float().abs().max().item()
    assert err <= (1e-2 if dtype != torch.float32 else 1e-5) * max(scale, 1e-6), (err, scale)


@pytest.mark.parametrize("case", EXPERT_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-N{c[2]}-k{c[3]}-{str(c[4]).split('.')[-1]}-{c[5]}")
def test_expert_segment_algorithm_equals_gather(case, device):
    """The expert-centric organisation (schedule -> coefficients per sorted pair -> token sum) uses
    the same per-pair arithmetic and the same summation order: bit-identical output."""
    T, H, N, k, dtype, kind = case
    d = [t.to(device) for t in _expert_inputs(T, H, N, k, dtype, kind, seed=T + H)]
    print(f"expert segment T={T} H={H} N={N} k={k} {dtype} {kind}", flush=True)
    a = _ops().hip_omni_expert_func(*d, algo="gather")
    b = _ops().hip_omni_expert_func(*d, algo="segment")
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.fixture(scope="module")
def config3_inputs():
    """benchmark config 3 at full size, exactly what bench.py times: 16384 tokens, hidden 1024, 4096 experts, k=16, bf16, seed 2;
    the oracle's output for all 16384 tokens (token chunks of 2048, fp32 sums, one rounding)."""
    T, H, N, k = 16384, 1024, 4096, 16
    x, up, down, gates, ids = oracle.make_expert_inputs(2, T, H, N, k)
    return (x, up, down, gates, ids), oracle.expert_forward(x, up, down, gates, ids)


@pytest.mark.parametrize("algo", ["auto", "split", "gather", "segment"])
def test_expert_config3_full_size(algo, config3_inputs, device):
    (x, up, down, gates, ids), want = config3_inputs
    print(f"expert config 3 full size, algo={algo}", flush=True)
    got = _ops().hip_omni_expert_func(*(t.to(device) for t in (x, up, down, gates, ids)), algo=algo)
    torch.cuda.synchronize()
    g, w = got.cpu().float(), want.float()
    torch.testing.assert_close(g, w, rtol=2e-2, atol=2e-2)
    # both sum in fp32 and round once: at most one bf16 ulp apart, on the scale of the output (max |y| ~ 0.02)
    scale = w.abs().max().item()
    assert (g - w).abs().max().item() <= 1e-2 * scale, ((g - w).abs().max().item(), scale)
    assert (g != w).float().mean().item() < 0.05          # and most elements are bit-identical


def _split_covers(H, dtype):
    """A row must cut into column blocks (1 .. 64 of them) of 8 slices of 64 .. 1024 bytes, a power of two."""
    es = torch.empty((), dtype=dtype).element_size()
    for b in range(1, 65):
        if H % b == 0 and (H // b) * es % 128 == 0 and (H // b) * es // 8 in (64, 128, 256, 512, 1024):
            return True
    return False


WIDE_ROW_CASES = [(96, 8192, 64, 8, torch.bfloat16, "ref"),      # 16 KiB rows: two column blocks of 8 x 1 KiB
                  (50, 6144, 32, 6, torch.bfloat16, "ref"),      # 12 KiB: three blocks of 8 x 512 B
                  (40, 4096, 32, 4, torch.float32, "ref"),       # fp32, 16 KiB
                  (33, 16384, 16, 2, torch.float16, "ref")]      # 32 KiB: four blocks


@pytest.mark.parametrize("case", WIDE_ROW_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-N{c[2]}-k{c[3]}-{str(c[4]).split('.')[-1]}")
def test_expert_rows_beyond_8_kib(case, device):
    """The reference puts no limit on the hidden size (omni_expert.py:920-992 tiles it).  Rows beyond 8 KiB, which the
    whole-row gather kernel cannot hold in registers, go through the hidden-split kernels in column blocks; that is also what
    AUTO picks for them."""
    T, H, N, k, dtype, kind = case
    x, up, down, gates, ids = _expert_inputs(T, H, N, k, dtype, kind, seed=T + H)
    if dtype == torch.float16:
        x, up = x * 0.25, up * 0.25                        # keep 16384-term dot products well inside f16's range of interest
    d = [t.to(device) for t in (x, up, down, gates, ids)]
    print(f"expert wide rows T={T} H={H} N={N} k={k} {dtype}", flush=True)
    want = oracle.expert_forward(x, up, down, gates, ids)
    got = _ops().hip_omni_expert_func(*d)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))
    scale = max(want.float().abs().max().item(), 1e-6)
    assert (got.cpu().float() - want.float()).abs().max().item() <= (1e-2 if dtype != torch.float32 else 1e-5) * scale
    assert torch.equal(got, _ops().hip_omni_expert_func(*d, algo="split"))
    with pytest.raises(ValueError):                        # the whole-row kernels refuse such rows by name
        _ops().hip_omni_expert_func(*d, algo="gather")


@pytest.mark.parametrize("case", EXPERT_CASES + [(4100, 1024, 4096, 16, torch.bfloat16, "ref"), (1000, 256, 512, 10, torch.float16, "ref"),
                                                 (130, 512, 64, 34, torch.float32, "ref"), (64, 4096, 16, 128, torch.bfloat16, "ref")],
                         ids=lambda c: f"T{c[0]}-H{c[1]}-N{c[2]}-k{c[3]}-{str(c[4]).split('.')[-1]}-{c[5]}")
def test_expert_split_algorithm(case, device):
    """The hidden-split organisation (8 column slices, one per XCD, partial dot products summed in slice order):
    same tolerance against the oracle, agreement with the gather algorithm to fp32 rounding, run-to-run identical;
    rows that do not cut into 8 power-of-two slices are refused."""
    T, H, N, k, dtype, kind = case
    x, up, down, gates, ids = _expert_inputs(T, H, N, k, dtype, kind, seed=T + H)
    d = [t.to(device) for t in (x, up, down, gates, ids)]
    print(f"expert split T={T} H={H} N={N} k={k} {dtype} {kind}", flush=True)
    if not _split_covers(H, dtype):
        with pytest.raises(ValueError):
            _ops().hip_omni_expert_func(*d, algo="split")
        return
    got = _ops().hip_omni_expert_func(*d, algo="split")
    assert torch.equal(got, _ops().hip_omni_expert_func(*d, algo="split"))
    want = oracle.expert_forward(x, up, down, gates, ids)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))
    ref = _ops().hip_omni_expert_func(*d, algo="gather").float()
    scale = max(ref.abs().max().item(), 1e-6)
    # one storage ulp at most where the fp32 sums straddle a rounding boundary
    assert (got.float() - ref).abs().max().item() <= (1e-2 if dtype != torch.float32 else 1e-5) * scale


def test_expert_split_tables_beyond_4gib(device):
    """Tables of 4 GiB each: the split kernels then take their 64-bit row offsets (below that size they use 32-bit ones).
    Rows built on the device, ids from both ends of the tables; checked against the oracle on the rows that are used."""
    T, H, N, k = 256, 2048, 1 << 20, 8
    g = torch.Generator().manual_seed(11)
    print(f"expert split 4 GiB tables T={T} H={H} N={N} k={k}", flush=True)
    up = torch.empty(N, H, dtype=torch.bfloat16, device=device).normal_(0, 0.05)
    down = torch.empty(N, H, dtype=torch.bfloat16, device=device).normal_(0, 0.05)
    x = (torch.randn(T, H, generator=g) * 0.5).bfloat16()
    gates = torch.rand(T, k, generator=g).bfloat16()
    ids = torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)
    ids[:, 0] = N - 1 - torch.arange(T, dtype=torch.int32)            # the far end: byte offsets beyond 2^32
    ids[:, 1] = torch.arange(T, dtype=torch.int32)
    d = [x.to(device), up, down, gates.to(device), ids.to(device)]
    got = _ops().hip_omni_expert_func(*d, algo="split")
    ref = _ops().hip_omni_expert_func(*d, algo="gather")
    # the oracle on a compact copy of the rows in use
    used, inv = torch.unique(ids.long(), return_inverse=True)
    want = oracle.expert_forward(x, up[used.to(device)].cpu(), down[used.to(device)].cpu(), gates, inv.int())
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(torch.bfloat16))
    scale = max(ref.float().abs().max().item(), 1e-6)
    assert (got.float() - ref.float()).abs().max().item() <= 1e-2 * scale
    del up, down
    torch.cuda.empty_cache()


DENSE_CASES = [(16384, 1024, 256, 16, torch.bfloat16, "baseline"),   # the shape the build plan names for the group regime: 1024 pairs per expert
               (4096, 512, 64, 8, torch.bfloat16, "ref"),              # negative gates, ids with replacement (duplicates add)
               (2048, 256, 32, 6, torch.float16, "ref"),
               (1000, 1024, 96, 10, torch.bfloat16, "ref"),            # ragged token count, N a multiple of 32 only
               (333, 64, 2048, 4, torch.bfloat16, "ref")]              # sparse use of the largest table the algorithm takes


@pytest.mark.parametrize("case", DENSE_CASES, ids=lambda c: f"T{c[0]}-H{c[1]}-N{c[2]}-k{c[3]}-{str(c[4]).split('.')[-1]}-{c[5]}")
def test_expert_dense_algorithm(case, device):
    """The dense organisation for the reference's group regime (T*k/N > 256, omni_scheduler.py:58): a gate matrix and two
    MFMA GEMMs over all experts.  Same tolerance against the oracle; agreement with the gather algorithm to the 16
    significant bits its coefficients carry; run-to-run identical; AUTO never picks it (it touches unselected rows)."""
    from omni_moe.ops.hip import _lib
    T, H, N, k, dtype, kind = case
    x, up, down, gates, ids = _expert_inputs(T, H, N, k, dtype, kind, seed=T + H)
    d = [t.to(device) for t in (x, up, down, gates, ids)]
    print(f"expert dense T={T} H={H} N={N} k={k} {dtype} {kind}", flush=True)
    got = _ops().hip_omni_expert_func(*d, algo="dense")
    assert torch.equal(got, _ops().hip_omni_expert_func(*d, algo="dense"))
    want = oracle.expert_forward(x, up, down, gates, ids)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))
    ref = _ops().hip_omni_expert_func(*d, algo="gather").float()
    scale = max(ref.abs().max().item(), 1e-6)
    assert (got.float() - ref).abs().max().item() <= 1e-2 * scale          # one storage ulp where the sums straddle a rounding boundary
    assert (got.float() != ref).float().mean().item() < 0.05
    lib = _lib.load()
    auto_ws = lib.omni_expert_workspace_bytes(T, H, N, k, _lib.DTYPE_CODE[dtype], _lib.ALGO_AUTO)
    dense_ws = lib.omni_expert_workspace_bytes(T, H, N, k, _lib.DTYPE_CODE[dtype], _lib.ALGO_DENSE)
    assert dense_ws > 0 and auto_ws != dense_ws          # by name only


def test_expert_unselected_nonfinite_rows(device):
    """A table row that no token selects may hold anything: the reference only ever touches selected rows
    (omni_expert.py:8-168 walks the scheduled pairs), and so do the gather, split and segment algorithms and
    whatever AUTO picks -- also in the group regime (T*k/N > 256), where AUTO used to switch to the dense
    algorithm.  The dense algorithm, by name, multiplies every token by every row: an Inf in an unselected
    down row reaches every token (0 * Inf), which is the documented difference that keeps it out of AUTO."""
    hip = _ops()
    T, H, N, k = 8192, 256, 64, 8                          # 1024 pairs per expert: the group regime
    g = torch.Generator().manual_seed(31)
    x = torch.randn(T, H, generator=g).bfloat16()
    up, down = ((torch.randn(N, H, generator=g) * 0.1).bfloat16() for _ in range(2))
    gates = torch.rand(T, k, generator=g).bfloat16()
    ids = torch.randint(0, N - 2, (T, k), generator=g, dtype=torch.int32)       # rows N-2 and N-1 are never selected
    want = oracle.expert_forward(x, up, down, gates, ids)
    up[N - 2, 5], up[N - 2, 9] = float("inf"), float("nan")
    down[N - 1, 7] = float("inf")
    d = [t.to(device) for t in (x, up, down, gates, ids)]
    print("expert op with non-finite unselected rows", flush=True)
    for algo in ("auto", "gather", "split", "segment"):
        got = hip.hip_omni_expert_func(*d, algo=algo).cpu().float()
        assert torch.isfinite(got).all(), algo
        torch.testing.assert_close(got, want.float(), rtol=2e-2, atol=2e-2)
    dense = hip.hip_omni_expert_func(*d, algo="dense").cpu().float()
    assert not torch.isfinite(dense[:, 7]).any()           # the unselected Inf row poisons column 7 of every token
    cols = [c for c in range(H) if c != 7]
    torch.testing.assert_close(dense[:, cols], want.float()[:, cols], rtol=2e-2, atol=2e-2)   # the up-table Inf/NaN is masked by the zero gate


def test_expert_dense_refusals_and_bad_ids(device):
    hip = _ops()
    x, up, down, gates, ids = (t.to(device) for t in _expert_inputs(64, 128, 48, 4, torch.bfloat16, "ref", 3))
    with pytest.raises(ValueError):                       # 48 experts: not a multiple of 32
        hip.hip_omni_expert_func(x, up, down, gates, ids, algo="dense")
    x, up, down, gates, ids = (t.to(device) for t in _expert_inputs(64, 128, 64, 4, torch.float32, "ref", 3))
    with pytest.raises(ValueError):                       # fp32 storage
        hip.hip_omni_expert_func(x, up, down, gates, ids, algo="dense")
    g = torch.Generator().manual_seed(5)
    T, H, N, k = 3000, 512, 128, 8
    x, up, down = torch.randn(T, H, generator=g).bfloat16(), (torch.randn(N, H, generator=g) * 0.05).bfloat16(), (torch.randn(N, H, generator=g) * 0.05).bfloat16()
    gates = torch.rand(T, k, generator=g).bfloat16()
    ids = torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)
    ids[::7, 3] = N + 5                                    # ids outside the table contribute nothing
    ids[::11, 0] = -1
    ok = (ids >= 0) & (ids < N)
    want = oracle.expert_forward(x, up, down, torch.where(ok, gates, torch.zeros_like(gates)), torch.where(ok, ids, torch.zeros_like(ids)))
    got = hip.hip_omni_expert_func(*(t.to(device) for t in (x, up, down, gates, ids)), algo="dense")
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=2e-2, atol=2e-2)
    y0 = hip.hip_omni_expert_func(x.to(device), up.to(device), down.to(device), gates[:, :0].to(device), ids[:, :0].to(device), algo="dense")
    assert torch.count_nonzero(y0).item() == 0             # k = 0 -> zeros


def test_expert_split_bad_ids(device):
    g = torch.Generator().manual_seed(12)
    T, H, N, k = 2100, 1024, 512, 8
    x, up, down = torch.randn(T, H, generator=g).bfloat16(), (torch.randn(N, H, generator=g) * 0.05).bfloat16(), (torch.randn(N, H, generator=g) * 0.05).bfloat16()
    gates = torch.rand(T, k, generator=g).bfloat16()
    ids = torch.randint(0, N, (T, k), generator=g, dtype=torch.int32)
    ids[::7, 3] = N + 5
    ids[::11, 0] = -1
    ok = (ids >= 0) & (ids < N)
    want = oracle.expert_forward(x, up, down, torch.where(ok, gates, torch.zeros_like(gates)), torch.where(ok, ids, torch.zeros_like(ids)))
    got = _ops().hip_omni_expert_func(*(t.to(device) for t in (x, up, down, gates, ids)), algo="split")
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=2e-2, atol=2e-2)


def test_expert_segment_skewed_and_bad_ids(device):
    g = torch.Generator().manual_seed(11)
    T, H, N, k = 4096, 1024, 512, 8
    x, up, down = torch.randn(T, H, generator=g).bfloat16(), (torch.randn(N, H, generator=g) * 0.05).bfloat16(), (torch.randn(N, H, generator=g) * 0.05).bfloat16()
    gates = torch.rand(T, k, generator=g).bfloat16()
    w = 1.0 / torch.arange(1, N + 1, dtype=torch.float64) ** 1.5            # one very hot expert
    ids = torch.multinomial(w, T * k, replacement=True, generator=g).reshape(T, k).to(torch.int32)
    ids[::7, 3] = N + 5                                                      # ids outside the table contribute nothing
    ids[::11, 0] = -1
    d = [t.to(device) for t in (x, up, down, gates, ids)]
    a = _ops().hip_omni_expert_func(*d, algo="gather")
    b = _ops().hip_omni_expert_func(*d, algo="segment")
    assert torch.equal(a, b)
    ok = (ids >= 0) & (ids < N)
    want = oracle.expert_forward(x, up, down, torch.where(ok, gates, torch.zeros_like(gates)), torch.where(ok, ids, torch.zeros_like(ids)))
    torch.testing.assert_close(a.cpu().float(), want.float(), rtol=2e-2, atol=2e-2)


def test_expert_edge_cases(device):
    hip = _ops()
    x, up, down, gates, ids = (t.to(device) for t in _expert_inputs(16, 256, 32, 4, torch.bfloat16, "ref", 1))
    assert hip.hip_omni_expert_func(x[:0], up, down, gates[:0], ids[:0]).shape == (0, 256)       # no tokens
    y0 = hip.hip_omni_expert_func(x, up, down, gates[:, :0], ids[:, :0])                         # k = 0 -> zeros
    assert torch.count_nonzero(y0).item() == 0
    y1 = hip.hip_omni_expert_func(x, up, down, gates, ids)
    y2 = hip.hip_omni_expert_func(x, up, down, gates, ids)
    assert torch.equal(y1, y2)                                                                   # deterministic
    perm = torch.tensor([2, 0, 3, 1], device=device)
    y3 = hip.hip_omni_expert_func(x, up, down, gates[:, perm].contiguous(), ids[:, perm].contiguous())
    torch.testing.assert_close(y3.float(), y1.float(), rtol=2e-2, atol=1e-3)                     # slot order is free
    with pytest.raises(ValueError):
        hip.hip_omni_expert_func(x, up, down[:, :128], gates, ids)


def test_schedule_drops_out_of_range_ids(device):
    g = torch.Generator().manual_seed(9)
    T, k, N = 300, 6, 50
    ids = torch.randint(-3, N + 5, (T, k), generator=g, dtype=torch.int32)
    got = _ops().hip_omni_schedule_func(ids.to(device), N)
    flat = ids.reshape(-1)
    valid = (flat >= 0) & (flat < N)
    want_off = torch.zeros(N + 1, dtype=torch.int64)
    want_off[1:] = torch.cumsum(torch.bincount(flat[valid].long(), minlength=N), 0)
    assert torch.equal(got.offsets.cpu().long(), want_off)
    nv = int(valid.sum())
    pairs = got.sorted_pair_ids.cpu().long()
    order = torch.sort(torch.where(valid, flat, torch.full_like(flat, N)).long(), stable=True).indices
    assert torch.equal(pairs[:nv], order[:nv])
    assert torch.equal(torch.sort(pairs).values, torch.arange(T * k))       # still a permutation


@pytest.mark.parametrize("algo", ["gather", "segment", "split"])
def test_expert_unused_rows_may_hold_nan(algo, device):
    """Padded slots and ids outside the table stand in for row 0 when rows are fetched; whatever row 0 holds must not
    leak: with NaN in the rows of experts that no valid pair selects, every output stays finite and unchanged."""
    T, H, N, k = 2100, 256, 2048, 6                                # k is no multiple of any batch size
    x, up, down, gates, ids = _expert_inputs(T, H, N, k, torch.bfloat16, "ref", seed=5)
    ids = ids.clamp(min=1)                                         # nobody selects expert 0 ...
    ids[::9, 2] = N + 1                                            # ... and some ids fall outside the table
    d = [t.to(device) for t in (x, up, down, gates, ids)]
    want = _ops().hip_omni_expert_func(*d, algo=algo)
    up2, down2 = up.clone(), down.clone()
    up2[0], down2[0] = float("nan"), float("inf")
    got = _ops().hip_omni_expert_func(d[0], up2.to(device), down2.to(device), d[3], d[4], algo=algo)
    assert torch.isfinite(got).all() and torch.equal(got, want)
