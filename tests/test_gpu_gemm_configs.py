"""GPU parity at the full sizes of the five benchmark configurations, through the C ABI.

Where the fp64 oracle finishes in seconds the whole matrix is compared (C1, C2, C4).  At 8192^3 and at K=65536 the
check is size-independent: Freivalds' identity C x = A (B x) over the whole matrix in fp64, the exact oracle on sampled
rows and columns that include every tile boundary, a full on-device comparison against the independent baseline kernel,
and the reference driver's known-answer inputs (tiled numbers x identity must reproduce A exactly).
"""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

TOL = 1e-3  # normalised max error, fp32 accumulate vs fp64 oracle

SEED_A, SEED_B = 20010106, 19980724

CONFIGS = {
    # name: (M, N, K, dtype, data code, param)
    "c1": (512, 512, 512, 0, 3, 1.0),
    "c2": (4096, 4096, 4096, 0, 3, 1.0),
    "c3": (8192, 8192, 8192, 1, 4, 8192 ** -0.5),
    "c4": (16384, 128, 8192, 0, 3, 1.0),
    "c5": (2048, 2048, 65536, 0, 3, 0.5),
}


def _inputs(name):
    M, N, K, dtype, code, param = CONFIGS[name]
    a = H.gen_on_device(M, K, code, False, dtype, param, SEED_A)
    b = H.gen_on_device(N, K, code, True, dtype, param, SEED_B)
    return M, N, K, dtype, a, b


def _device_baseline_rel_err(gpu, M, N, K, a, b, c, dtype):
    cb = H.poisoned_c(M, N)
    gpu.matmul_baseline(H.tensors(M, N, K, a, b, cb, dtype), H.stream_handle())
    res = torch.zeros(4, dtype=torch.int64, device="cuda")
    gpu.compare_tensors(cb.data_ptr(), c.data_ptr(), M, N, res.data_ptr(), H.stream_handle())
    torch.cuda.synchronize()
    r = res.cpu().numpy().view(np.uint64)
    diff = np.array([r[1]]).view(np.float64)[0]
    ref = np.array([r[2]]).view(np.float64)[0]
    return diff / ref


@pytest.mark.parametrize("name", ["c1", "c2", "c4"])
def test_config_full_matrix_vs_oracle(gpu, oracle, name):
    M, N, K, dtype, a, b = _inputs(name)
    c = H.run_mfma(M, N, K, a, b, dtype)
    ha, hb = H.to_host_u16(a), H.to_host_u16(b)
    ref = oracle.gemm_f64(M, N, K, ha, hb, dtype)
    absref = oracle.gemm_f64(M, N, K, ha, hb, dtype, abs_mode=True)
    m = oracle.error_metrics(c.cpu().numpy(), ref, absref)
    print(name, gpu.matmul_mfma_plan(H.tensors(M, N, K, a, b, c, dtype)), m)
    assert m["max_rel_err"] < TOL
    # componentwise: |err| <= K * 2^-24 * sum_k |a||b| is the worst case of fp32 accumulation
    assert m["max_componentwise"] < K * 2.0 ** -24


@pytest.mark.parametrize("name", ["c3", "c5"])
def test_config_sampled_oracle_freivalds_and_device_baseline(gpu, oracle, name):
    M, N, K, dtype, a, b = _inputs(name)
    c = H.run_mfma(M, N, K, a, b, dtype)
    plan = gpu.matmul_mfma_plan(H.tensors(M, N, K, a, b, c, dtype))
    ha, hb, hc = H.to_host_u16(a), H.to_host_u16(b), c.cpu().numpy()
    # rows/cols on both sides of every 64-row tile boundary (covers 64/128/256 tiles) plus seeded random ones
    rng = np.random.default_rng(7)
    edges = np.arange(0, M, 256)
    rows = np.unique(np.concatenate([edges, edges + 255, rng.integers(0, M, 16)]))[:96]
    ref_rows = oracle.gemm_f64_rows(M, N, K, ha, hb, dtype, rows)
    scale = np.abs(ref_rows).max()
    err_rows = np.abs(hc[rows].astype(np.float64) - ref_rows).max() / scale
    edges = np.arange(0, N, 256)
    cols = np.unique(np.concatenate([edges, edges + 255, rng.integers(0, N, 16)]))[:96]
    ref_cols = oracle.gemm_f64_cols(M, N, K, ha, hb, dtype, cols)
    err_cols = np.abs(hc[:, cols].astype(np.float64) - ref_cols).max() / scale
    resid, fscale = oracle.freivalds(M, N, K, ha, hb, hc, dtype, n_vec=4)
    dev = _device_baseline_rel_err(gpu, M, N, K, a, b, c, dtype)
    print(name, plan, "rows", err_rows, "cols", err_cols, "freivalds", (resid / fscale).max(), "device baseline", dev)
    assert err_rows < TOL and err_cols < TOL
    # |C x - A(B x)| is a sum of N rounding errors each bounded by K 2^-24 sum|a||b|: far below 1e-3 of the scale
    assert (resid / fscale).max() < 1e-4
    assert dev < TOL


def test_deep_k_config_as_benchmarked_with_the_preferred_workspace(gpu, oracle):
    """C5 the way the benchmark runs it: with the workspace the planner prefers, which makes it four K partitions of
    256x256 tiles summed from copies of C.  Checked against the oracle on sampled rows and against the device baseline
    over the whole matrix; summed by a launch of its own and inside the GEMM launch the bits must be the same; stream-K
    with the same room must be as accurate."""
    M, N, K, dtype, a, b = _inputs("c5")
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype)
    _, pref = gpu.matmul_mfma_workspace_bytes_for(t)
    ws = torch.empty(pref, dtype=torch.uint8, device="cuda")
    plan = gpu.matmul_mfma_describe(t, workspace_bytes=pref)
    assert "split k (workspace sum)" in plan, plan
    results = []
    for in_launch in (False, True):
        c.view(torch.uint8).fill_(0x7D)
        ws.fill_(0xFF)
        was, _ = gpu.matmul_mfma_sum_in_launch(in_launch)
        try:
            gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
        finally:
            gpu.matmul_mfma_sum_in_launch(was)
        torch.cuda.synchronize()
        results.append(c.clone())
    assert torch.equal(results[0], results[1])
    ha, hb = H.to_host_u16(a), H.to_host_u16(b)
    rng = np.random.default_rng(11)
    edges = np.arange(0, M, 256)
    rows = np.unique(np.concatenate([edges, edges + 255, rng.integers(0, M, 16)]))[:32]
    ref_rows = oracle.gemm_f64_rows(M, N, K, ha, hb, dtype, rows)
    err_rows = np.abs(results[0][rows].cpu().numpy().astype(np.float64) - ref_rows).max() / np.abs(ref_rows).max()
    dev = _device_baseline_rel_err(gpu, M, N, K, a, b, results[0], dtype)
    c.view(torch.uint8).fill_(0x7D)
    gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, gpu.K_STREAM, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    dev_stream = _device_baseline_rel_err(gpu, M, N, K, a, b, c, dtype)
    print(plan, "rows", err_rows, "device baseline", dev, "stream-K", dev_stream)
    assert err_rows < TOL and dev < TOL and dev_stream < TOL


def test_headline_known_answer_tiled_times_identity(gpu, oracle):
    """gemm/gemm_main.cpp:81-85 at the headline size: C must reproduce A exactly."""
    M = N = K = 8192
    for dtype in (0, 1):
        a, b = H.make_inputs(M, N, K, dtype, 2, 1)
        c = H.run_mfma(M, N, K, a, b, dtype)
        a_f32 = torch.from_numpy(oracle.widen(H.to_host_u16(a), dtype)).cuda()
        assert torch.equal(c, a_f32)


def test_every_tile_and_split_on_headline_shape(gpu):
    """Each tile of the family, output stationary and split-K, against the device baseline at 8192^3 bf16."""
    M, N, K, dtype, a, b = _inputs("c3")
    assert gpu.tile_count() >= 14
    for tile in range(1, gpu.tile_count()):
        for k_mode in (gpu.K_OUTPUT_STATIONARY, gpu.K_SPLIT):
            c = H.run_mfma(M, N, K, a, b, dtype, k_mode, tile)
            assert _device_baseline_rel_err(gpu, M, N, K, a, b, c, dtype) < TOL, (tile, k_mode)


@pytest.mark.parametrize("shape", [(128, 1_000_000, 72), (1_000_000, 96, 136), (200, 70_001 * 8, 64)])
def test_extreme_aspect_ratios(gpu, oracle, shape):
    """A million rows or columns with a short K: every index computation of the kernel (tile ids, 32-bit buffer
    offsets, row pitches of C up to 4 MB) at the far end of its range.  Whole-matrix comparison against the baseline
    kernel on the device, the exact oracle on sampled rows and columns including the last ones."""
    M, N, K = shape
    dtype = 1
    a = H.gen_on_device(M, K, 3, False, dtype, 1.0, SEED_A)
    b = H.gen_on_device(N, K, 3, True, dtype, 1.0, SEED_B)
    c = H.run_mfma(M, N, K, a, b, dtype)
    assert _device_baseline_rel_err(gpu, M, N, K, a, b, c, dtype) < 1e-5
    ha, hb = H.to_host_u16(a), H.to_host_u16(b)
    hc = c.cpu().numpy()
    rows = np.unique(np.array([0, 1, M // 2, M - 2, M - 1], dtype=np.uint32))
    cols = np.unique(np.array([0, 1, N // 3, N - 2, N - 1], dtype=np.uint32))
    ref_rows = oracle.gemm_f64_rows(M, N, K, ha, hb, dtype, rows)
    ref_cols = oracle.gemm_f64_cols(M, N, K, ha, hb, dtype, cols)
    scale = max(np.abs(ref_rows).max(), np.abs(ref_cols).max())
    assert np.abs(hc[rows] - ref_rows).max() / scale < TOL
    assert np.abs(hc[:, cols] - ref_cols).max() / scale < TOL


PEELED = [
    # (M, N, K, c_col_major, what the plan must contain).  A few rows or columns over a multiple of the largest tile
    # on a problem of many tiles, or a tile column over a whole round: whatever the planner's constants, peeling wins
    # by a wide margin here.
    (8200, 8192, 2048, 0, ["peeled", " + bottom "]),
    (8192, 8200, 2048, 0, ["peeled", " + right "]),
    (8192, 8200, 2048, 1, ["peeled", " + bottom "]),                  # column-major C: operands swap, so does the strip
    (4104, 4104, 8192, 0, ["peeled", " + bottom ", " + right "]),      # 289 tiles of 256x256 would be a round and a bit
    (8200, 8192, 4104, 0, ["peeled", " + bottom ", "split k"]),       # ragged K too; the strip splits K through atomics
    (4096, 4352, 8192, 0, ["peeled", " + right 4096x256x8192"]),      # 272 tiles of 256x256: one round, then the rest
]


@pytest.mark.parametrize("case", PEELED)
def test_ragged_shapes_are_peeled_and_exact_to_tolerance(gpu, oracle, case):
    """A large problem whose M or N is a little over a multiple of the tile: the whole tiles run the plain kernel and
    the leftover rows and columns run as small range-checked launches into the same C (some with K split through
    atomics on a zero-filled strip).  Every element of C must be written, nothing outside it, and the result must
    match the fp64 oracle on rows and columns around the seams and the device baseline everywhere."""
    M, N, K, cc, wanted = case
    dtype = 1
    a = H.gen_on_device(M, K, 4, False, dtype, K ** -0.5, SEED_A)
    b = H.gen_on_device(N, K, 4, True, dtype, K ** -0.5, SEED_B)
    guard = 1 << 16
    buf = torch.empty(M * N + 2 * guard, dtype=torch.float32, device="cuda")
    buf.fill_(float("nan"))
    c = buf[guard:guard + M * N].view((N, M) if cc else (M, N))
    t = H.tensors(M, N, K, a, b, c, dtype, 0, 1, cc)
    text = gpu.matmul_mfma_describe(t)
    for w in wanted:
        assert w in text, text
    gpu.matmul_mfma(t, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    assert bool(torch.isnan(buf[:guard]).all()) and bool(torch.isnan(buf[guard + M * N:]).all()), "stored outside C"
    got = c.t() if cc else c
    assert not bool(torch.isnan(got).any()), "an element of C was never written"
    ha, hb = H.to_host_u16(a), H.to_host_u16(b)
    hc = got.cpu().numpy()
    rows = np.unique(np.clip(np.array([0, 255, 256, M // 256 * 256 - 1, M // 256 * 256, M - 1, M // 2]), 0, M - 1))
    ref_rows = oracle.gemm_f64_rows(M, N, K, ha, hb, dtype, rows)
    scale = np.abs(ref_rows).max()
    assert np.abs(hc[rows].astype(np.float64) - ref_rows).max() / scale < TOL
    cols = np.unique(np.clip(np.array([0, 255, 256, N // 256 * 256 - 1, N // 256 * 256, N - 1, N // 2]), 0, N - 1))
    ref_cols = oracle.gemm_f64_cols(M, N, K, ha, hb, dtype, cols)
    assert np.abs(hc[:, cols].astype(np.float64) - ref_cols).max() / scale < TOL
    if not cc:
        assert _device_baseline_rel_err(gpu, M, N, K, a, b, c, dtype) < TOL
    # a forced tile is one range-checked launch over everything: same numbers to rounding
    c2 = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    gpu.matmul_mfma(H.tensors(M, N, K, a, b, c2, dtype, 0, 1, cc), gpu.K_OUTPUT_STATIONARY, gpu.TILE_128x128, H.stream_handle())
    torch.cuda.synchronize()
    assert float((c2 - c).abs().max()) / scale < 1e-5


READ_ONCE = [
    # (M, N, K, c_col_major, forced tile, K mode, the operand the plan must name).  One operand of 257 MiB, the other
    # dimension one tile: every workgroup reads its own slice of the large operand and all of the small one.
    (256, 8192, 16448, 0, "TILE_256x128", "K_OUTPUT_STATIONARY", "B non-temporal"),
    (256, 8192, 16448, 0, "TILE_256x256", "K_SPLIT_REDUCE", "B non-temporal"),
    (192, 8192, 16448, 0, "TILE_192x256", "K_OUTPUT_STATIONARY", "B non-temporal"),
    (8192, 256, 16448, 0, "TILE_256x256", "K_OUTPUT_STATIONARY", "A non-temporal"),
    (8192, 192, 16448, 0, "TILE_256x192", "K_SPLIT_REDUCE", "A non-temporal"),
    (8192, 256, 16448, 1, "TILE_256x256", "K_OUTPUT_STATIONARY", "B non-temporal"),   # column-major C swaps the operands
    (64, 8192 + 128, 16448, 0, "TILE_64x128", "K_OUTPUT_STATIONARY", "B non-temporal"),
    (256, 8192, 16448, 0, "TILE_AUTO", "K_AUTO", "B non-temporal"),
    (256, 8192, 16448, 0, "TILE_256x128", "K_SPLIT", "B non-temporal"),          # K partitions meeting through atomics
    (8192, 128, 16448, 0, "TILE_128x128", "K_SPLIT", "A non-temporal"),
]


@pytest.mark.parametrize("case", READ_ONCE)
def test_operand_read_once_is_streamed_non_temporal(gpu, oracle, case):
    """A problem one tile high (or wide) whose other operand is larger than the memory-side cache runs the build whose
    DMA of that operand is non-temporal.  Same numbers as the ordinary build to rounding, and the fp64 oracle on
    sampled rows and columns; builds without such a twin (range-checked, stream-K) and smaller operands keep the
    ordinary path."""
    M, N, K, cc, tile, k_mode, wanted = case
    dtype = 1
    a = H.gen_on_device(M, K, 4, False, dtype, K ** -0.5, SEED_A)
    b = H.gen_on_device(N, K, 4, True, dtype, K ** -0.5, SEED_B)
    ws = torch.empty(1 << 28, dtype=torch.uint8, device="cuda")
    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype, 0, 1, cc)
    text = gpu.matmul_mfma_describe(t, getattr(gpu, k_mode), getattr(gpu, tile), ws.numel())
    assert wanted in text, text
    gpu.matmul_mfma_ws(t, ws.data_ptr(), ws.numel(), getattr(gpu, k_mode), getattr(gpu, tile), H.stream_handle())
    torch.cuda.synchronize()
    got = c.t() if cc else c
    ha, hb = H.to_host_u16(a), H.to_host_u16(b)
    hc = got.cpu().numpy()
    rows = np.unique(np.clip(np.array([0, 63, 64, 127, 128, 255, 256, M - 1, M // 2, M // 2 + 1]), 0, M - 1))
    ref_rows = oracle.gemm_f64_rows(M, N, K, ha, hb, dtype, rows)
    scale = np.abs(ref_rows).max()
    assert np.abs(hc[rows].astype(np.float64) - ref_rows).max() / scale < TOL
    cols = np.unique(np.clip(np.array([0, 127, 128, 255, 256, N - 1, N // 2, N // 2 + 1]), 0, N - 1))
    ref_cols = oracle.gemm_f64_cols(M, N, K, ha, hb, dtype, cols)
    assert np.abs(hc[:, cols].astype(np.float64) - ref_cols).max() / scale < TOL
    # the 128x128 tile makes the problem two tiles high (or wide): the ordinary build, same numbers to rounding
    if min(M, N) > 128:
        c2 = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
        t2 = H.tensors(M, N, K, a, b, c2, dtype, 0, 1, cc)
        assert "non-temporal" not in gpu.matmul_mfma_describe(t2, gpu.K_OUTPUT_STATIONARY, gpu.TILE_128x128)
        gpu.matmul_mfma(t2, gpu.K_OUTPUT_STATIONARY, gpu.TILE_128x128, H.stream_handle())
        torch.cuda.synchronize()
        assert float((c2 - c).abs().max()) / scale < 1e-5


@pytest.mark.parametrize("entry", ["sm90", "sm80"])
def test_fp32_entry_points_at_the_headline_size(gpu, entry):
    """The Exo-named fp32 entry points (xgemm_Sm90.py:43-48 as the harness calls it, gemm/gemm_test.cu:335; xgemm_Sm80.py:18-21)
    at 8192^3 on normal(0,1)/sqrt(K) fp32 data: Freivalds' identity C x = A (B x) over the whole matrix in float64 for
    four random +-1 vectors, and sampled rows against numpy's float64 product, at the three-term bar (3e-5 of the
    scale: each operand carries 16 significant bits)."""
    M = N = K = 8192
    g = torch.Generator(device="cuda").manual_seed(8192)
    a = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32) * K ** -0.5
    b_nk = torch.randn((N, K), generator=g, device="cuda", dtype=torch.float32) * K ** -0.5   # B stored N x K
    c = H.poisoned_c(M, N)
    need = gpu.xgemm_workspace_bytes(1, M, N, K, gpu.F32_BF16X3)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ctxt = gpu.XgemmContext(ws.data_ptr(), need, H.stream_handle(), gpu.F32_BF16X3, gpu.TILE_AUTO)
    if entry == "sm90":
        # operands swapped, so that the proc's C[L,N,M] is the row-major M x N
        gpu.xgemm_Sm90_wgmma(ctxt, 1, N, M, 1, K, b_nk.data_ptr(), a.data_ptr(), c.data_ptr())
    else:
        b_kn = b_nk.t().contiguous()
        gpu.xgemm_Sm80(ctxt, M, N, K, a.data_ptr(), b_kn.data_ptr(), c.data_ptr())
        del b_kn
    torch.cuda.synchronize()
    ha, hb, hc = a.cpu().numpy(), b_nk.cpu().numpy(), c.cpu().numpy()
    assert np.isfinite(hc).all()
    rng = np.random.default_rng(11)
    x = rng.choice([-1.0, 1.0], size=(N, 4))
    bx = hb.astype(np.float64).T @ x                                                                # K x 4
    want = ha.astype(np.float64) @ bx                                                               # M x 4
    got = hc.astype(np.float64) @ x
    scale = np.abs(ha).astype(np.float64) @ (np.abs(hb).astype(np.float64).T @ np.ones((N, 1)))      # sum |a||b| per row
    assert (np.abs(got - want) / scale).max() < 3e-5
    rows = np.unique(np.concatenate([np.arange(0, M, 256), np.arange(255, M, 256), rng.integers(0, M, 16)]))[:80]
    ref_rows = ha[rows].astype(np.float64) @ hb.astype(np.float64).T
    assert np.abs(hc[rows] - ref_rows).max() / np.abs(ref_rows).max() < 3e-5


@pytest.mark.parametrize("shape", [(70_000, 256, 32_768), (33_000, 33_000, 64), (256, 70_000, 32_768), (47_000, 47_000, 64)])
def test_operands_and_results_beyond_four_gigabytes(gpu, shape):
    """A of 4.6 GB, C of 4.4 GB, B of 4.6 GB, C of 2.2e9 elements: byte offsets past 2^32 in the panel bases and in C, element
    indices past 2^31.  Checked on the device in
    float64 (torch is the independent implementation here): Freivalds' identity over the whole matrix, and the rows at
    the far end of the large tensor against a direct product."""
    M, N, K = shape
    dtype = 1
    a = H.gen_on_device(M, K, 4, False, dtype, K ** -0.5, SEED_A)
    b = H.gen_on_device(N, K, 4, True, dtype, K ** -0.5, SEED_B)
    assert max(a.numel() * 2, b.numel() * 2, M * N * 4) > 1 << 32
    c = H.run_mfma(M, N, K, a, b, dtype)
    af, bf = a.view(torch.bfloat16), b.view(torch.bfloat16)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = (torch.randint(0, 2, (N, 4), generator=g, device="cuda") * 2 - 1).double()
    bx = bf.double().T @ x if N * K <= 1 << 28 else torch.cat([bf[:, k0:k0 + 4096].double().T @ x for k0 in range(0, K, 4096)])
    b_abs = bf.double().abs().sum(0) if N * K <= 1 << 28 else torch.cat([bf[:, k0:k0 + 4096].double().abs().sum(0) for k0 in range(0, K, 4096)])
    worst = 0.0
    for r0 in range(0, M, 2048):
        rows = slice(r0, min(M, r0 + 2048))
        want = af[rows].double() @ bx
        got = c[rows].double() @ x
        scale = af[rows].double().abs() @ b_abs
        worst = max(worst, float(((got - want).abs().max(1).values / scale).max()))
    assert worst < 1e-4, worst
    for r in (0, M // 2, M - 257, M - 1):
        ref = af[r].double() @ bf.double().T if N * K <= 1 << 28 else torch.cat([af[r].double() @ bf[n0:n0 + 4096].double().T for n0 in range(0, N, 4096)])
        assert float((c[r].double() - ref).abs().max() / ref.abs().max()) < TOL, r
    del a, b, c
    torch.cuda.empty_cache()


@pytest.mark.parametrize("k_mode", ["K_SPLIT", "K_SPLIT_REDUCE"])
def test_k_partitions_of_a_result_beyond_four_gigabytes(gpu, k_mode):
    """C of 4.4 GB with K partitions forced: the zero fill, the atomic epilogue, the partitions' copies of C in a
    workspace of two or more times that size and the pass that sums them all index past 2^32 bytes."""
    M, N, K, dtype = 33_000, 33_000, 1024, 1
    a = H.gen_on_device(M, K, 4, False, dtype, K ** -0.5, SEED_A)
    b = H.gen_on_device(N, K, 4, True, dtype, K ** -0.5, SEED_B)
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype)
    mode = getattr(gpu, k_mode)
    plan = gpu.matmul_mfma_plan(t, mode, gpu.TILE_256x256)
    assert plan["k_splits"] >= 2, plan
    if k_mode == "K_SPLIT":
        gpu.matmul_mfma(t, mode, gpu.TILE_256x256, H.stream_handle())
    else:
        required, preferred = gpu.matmul_mfma_workspace_bytes_for(t, mode, gpu.TILE_256x256)
        assert required >= 2 * M * N * 4
        ws = torch.empty(preferred, dtype=torch.uint8, device="cuda")
        gpu.matmul_mfma_ws(t, ws.data_ptr(), preferred, mode, gpu.TILE_256x256, H.stream_handle())
    torch.cuda.synchronize()
    af, bf = a.view(torch.bfloat16).double(), b.view(torch.bfloat16).double()
    worst = 0.0
    for r0 in list(range(0, M, 4096)) + [M - 300]:
        rows = slice(r0, min(M, r0 + 300))
        ref = af[rows] @ bf.T
        worst = max(worst, float((c[rows].double() - ref).abs().max() / ref.abs().max()))
    assert worst < TOL, worst


@pytest.mark.parametrize("shape", [(256, 256, (1 << 21) - 64), (64, 192, (1 << 21) - 8), (300, 130, 1_500_008)])
def test_deepest_k_the_library_accepts(gpu, shape):
    """K just under the library's bound of 2^21 (rows of 4 MB: the largest buffer offsets a tile's DMA forms), whole
    tiles and ragged, against torch's float64 product; K at the bound is refused."""
    M, N, K = shape
    dtype = 1
    a = H.gen_on_device(M, K, 4, False, dtype, K ** -0.5, SEED_A)
    b = H.gen_on_device(N, K, 4, True, dtype, K ** -0.5, SEED_B)
    c = H.run_mfma(M, N, K, a, b, dtype)
    ref = a.view(torch.bfloat16).double() @ b.view(torch.bfloat16).double().T
    assert float((c.double() - ref).abs().max() / ref.abs().max()) < TOL
    t = H.tensors(M, N, 1 << 21, a, b, c, dtype)
    assert not gpu.matmul_mfma_supports(t, gpu.K_AUTO, gpu.TILE_AUTO)


def test_deepest_k_of_the_fp32_entry(gpu):
    """Three bf16 terms triple the depth: fp32 K = 699 048 is a bf16 problem 2 097 144 deep, the deepest accepted."""
    M, N, K = 128, 192, 699_048
    g = torch.Generator(device="cuda").manual_seed(21)
    a = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32) * K ** -0.5
    b = torch.randn((N, K), generator=g, device="cuda", dtype=torch.float32) * K ** -0.5
    c = H.poisoned_c(M, N)
    t = gpu.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), gpu.F32, 0, 1, 0)
    need = gpu.matmul_f32_workspace_bytes(t, gpu.F32_BF16X3)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    gpu.matmul_f32_ws(t, ws.data_ptr(), need, gpu.F32_BF16X3, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    ref = a.double() @ b.double().T
    assert float((c.double() - ref).abs().max() / ref.abs().max()) < 3e-5
    deeper = gpu.GpuTensors.make(M, N, K + 8, a.data_ptr(), b.data_ptr(), c.data_ptr(), gpu.F32, 0, 1, 0)
    with pytest.raises(gpu.MiGemmError):
        gpu.matmul_f32_workspace_bytes(deeper, gpu.F32_BF16X3)
