"""GPU parity tests at sizes the CPU oracle finishes in seconds.  Every GEMM goes through the C ABI."""
import numpy as np
import pytest
import torch

import helpers as H
import spork_amd as S

pytestmark = pytest.mark.gpu

TOL = 1e-3  # max|C - oracle| / max|oracle|, fp32 accumulate vs fp64 oracle (the benchmark's stated tolerance)


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("code,param", [(0, 1.0), (1, 1.0), (2, 1.0), (3, 1.0), (3, 0.5), (4, 1.0 / 64)])
@pytest.mark.parametrize("transpose_rule", [False, True])
def test_device_generator_matches_oracle(gpu, oracle, dtype, code, param, transpose_rule):
    rows, cols = 96, 200
    dev = H.to_host_u16(H.gen_on_device(rows, cols, code, transpose_rule, dtype, param, 777))
    ref = oracle.fill(rows, cols, code, transpose_rule, dtype, param, 777)
    if code == 4:
        # Box-Muller goes through libm on the host and the device math library on the GPU: equal up to one
        # unit in the last place of the 16-bit format in rare rounding-boundary cases.
        a = oracle.widen(dev, dtype).astype(np.float64)
        b = oracle.widen(ref, dtype).astype(np.float64)
        assert (dev != ref).mean() < 1e-3
        np.testing.assert_allclose(a, b, rtol=2 ** -7 if dtype == 1 else 2 ** -10, atol=1e-7)
    else:
        np.testing.assert_array_equal(dev, ref)


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("shape", [(32, 32, 16), (64, 96, 48), (128, 64, 512)])
def test_mfma_direct_vs_oracle(gpu, oracle, dtype, shape):
    M, N, K = shape
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0)
    c = H.poisoned_c(M, N)
    gpu.matmul_mfma_direct(H.tensors(M, N, K, a, b, c, dtype), H.stream_handle())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    assert H.rel_err(c.cpu().numpy(), ref) < TOL


def test_mfma_direct_tiled_numbers_identity_exact(gpu, oracle):
    """A = tiled numbers, B = identity (gemm/gemm_main.cpp:81-85): C must equal A's leading N columns exactly, which
    pins the (row, column) placement of every accumulator register."""
    M, N, K = 64, 64, 64
    for dtype in (0, 1):
        a, b = H.make_inputs(M, N, K, dtype, 2, 1)
        c = H.poisoned_c(M, N)
        gpu.matmul_mfma_direct(H.tensors(M, N, K, a, b, c, dtype), H.stream_handle())
        torch.cuda.synchronize()
        expect = oracle.widen(H.to_host_u16(a), dtype)[:, :N]
        np.testing.assert_array_equal(c.cpu().numpy(), expect)


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("layout", [(a, b, c) for a in (0, 1) for b in (0, 1) for c in (0, 1)])
def test_baseline_all_layouts_ragged(gpu, oracle, dtype, layout):
    """All 8 col_major combinations (gemm/gemm_baseline.cu:129-168) on a shape no tile divides."""
    M, N, K = 150, 77, 203
    ac, bc, cc = layout
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0, ac, bc)
    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    gpu.matmul_baseline(H.tensors(M, N, K, a, b, c, dtype, ac, bc, cc), H.stream_handle())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype, ac, bc)
    got = c.cpu().numpy()
    got = got.T if cc else got
    assert H.rel_err(got, ref) < 1e-5


# every tile of the family, as the library itself lists it: (code, rows, columns)
TILES = [pytest.param(t["code"], t["bm"], t["bn"], id=t["name"]) for t in S.tiles()]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("tile,bm,bn", TILES)
@pytest.mark.parametrize("mt,nt,K", [(1, 1, 32), (1, 1, 64), (2, 1, 96), (1, 3, 160), (2, 2, 1024),
                                      (1, 2, 128), (2, 1, 192), (1, 1, 256), (1, 1, 320)])  # 1..5 K tiles per ring
def test_mfma_tiles_output_stationary(gpu, oracle, dtype, tile, bm, bn, mt, nt, K):
    M, N = bm * mt, bn * nt
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0)
    c = H.run_mfma(M, N, K, a, b, dtype, gpu.K_OUTPUT_STATIONARY, tile)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    assert H.rel_err(c.cpu().numpy(), ref) < TOL


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("tile,bm,bn", TILES)
def test_mfma_tiles_known_answers(gpu, oracle, dtype, tile, bm, bn):
    """The reference driver's structured inputs (gemm/gemm_main.cpp:81-90): tiled x identity and identity x tiled
    give C = A[:, :N] and C = B[:M, :] exactly; plus the reference's own sparse-random style under its ratio test."""
    M, N, K = 2 * bm, 2 * bn, 512
    a, b = H.make_inputs(M, N, K, dtype, 2, 1)
    c = H.run_mfma(M, N, K, a, b, dtype, gpu.K_OUTPUT_STATIONARY, tile).cpu().numpy()
    np.testing.assert_array_equal(c, oracle.widen(H.to_host_u16(a), dtype)[:, :N])
    a, b = H.make_inputs(M, N, K, dtype, 1, 2)
    c = H.run_mfma(M, N, K, a, b, dtype, gpu.K_OUTPUT_STATIONARY, tile).cpu().numpy()
    b_logical = oracle.widen(H.to_host_u16(b), dtype).T  # stored N x K -> logical K x N
    np.testing.assert_array_equal(c, b_logical[:M, :])
    a, b = H.make_inputs(M, N, K, dtype, 0, 0)
    c = H.run_mfma(M, N, K, a, b, dtype, gpu.K_OUTPUT_STATIONARY, tile).cpu().numpy()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    assert oracle.compare_ratio(ref.astype(np.float32), c) is None
    assert H.rel_err(c, ref) < TOL


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("tile,bm,bn", TILES)
def test_mfma_split_k_and_col_major_c(gpu, oracle, dtype, tile, bm, bn):
    M, N, K = max(bm, 128), 2 * bn, 2048  # M a multiple of 128 so the swapped (column-major C) problem has a tile too
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    c = H.run_mfma(M, N, K, a, b, dtype, gpu.K_SPLIT, tile)
    assert H.rel_err(c.cpu().numpy(), ref) < TOL
    # column-major C: the callee swaps operands (gemm/gemm_sm80.cu:516-539); the buffer then holds C^T row-major
    ct = H.run_mfma(M, N, K, a, b, dtype, gpu.K_OUTPUT_STATIONARY, gpu.TILE_AUTO, c_col_major=1)
    assert H.rel_err(ct.cpu().numpy().T, ref) < TOL


def test_mfma_auto_plan_runs_unfriendly_shapes(gpu, oracle):
    """AUTO must pick something valid for every shape a tile divides, including a single 128x128 tile."""
    for M, N, K in [(128, 128, 32), (384, 640, 96), (512, 512, 512)]:
        a, b = H.make_inputs(M, N, K, 0, 3, 3, 1.0)
        c = H.run_mfma(M, N, K, a, b, 0)
        ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), 0)
        assert H.rel_err(c.cpu().numpy(), ref) < TOL


RAGGED = [(1, 1, 8), (33, 65, 72), (160, 480, 816), (257, 129, 200), (300, 500, 1000), (255, 127, 2040), (64, 64, 64)]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("tile", list(range(14)))
@pytest.mark.parametrize("shape", RAGGED)
def test_mfma_ragged_shapes(gpu, oracle, dtype, tile, shape):
    """M, N not multiples of any tile and K only a multiple of 8 (the reference driver's 160x480x816 among them,
    gemm/gemm_main.cpp:106): rows and K chunks past the edge must read as zero and nothing may be stored outside C."""
    M, N, K = shape
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    # C sits inside a larger poisoned buffer so that any store outside it is caught
    guard = 4096
    buf = torch.empty(M * N + 2 * guard, dtype=torch.float32, device="cuda")
    buf.view(torch.uint8).fill_(0x7D)
    c = buf[guard:guard + M * N].view(M, N)
    for k_mode in (gpu.K_OUTPUT_STATIONARY, gpu.K_SPLIT):
        buf.view(torch.uint8).fill_(0x7D)
        t = H.tensors(M, N, K, a, b, c, dtype)
        gpu.matmul_mfma(t, k_mode, tile, H.stream_handle())
        torch.cuda.synchronize()
        assert H.rel_err(c.cpu().numpy(), ref) < TOL, gpu.matmul_mfma_plan(t, k_mode, tile)
        edges = torch.cat([buf[:guard], buf[guard + M * N:]]).view(torch.uint8)
        assert bool((edges == 0x7D).all()), "stored outside C"


def test_mfma_ragged_column_major_c(gpu, oracle):
    M, N, K = 200, 72, 136
    a, b = H.make_inputs(M, N, K, 1, 3, 3, 1.0)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), 1)
    ct = H.run_mfma(M, N, K, a, b, 1, gpu.K_AUTO, gpu.TILE_AUTO, c_col_major=1)
    assert H.rel_err(ct.cpu().numpy().T, ref) < TOL


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("layout", [(a, b, c) for a in (0, 1) for b in (0, 1) for c in (0, 1)])
@pytest.mark.parametrize("shape", [(150, 77, 203), (256, 384, 512), (1000, 130, 66)])
def test_mfma_ws_all_layouts_any_k(gpu, oracle, dtype, layout, shape):
    """All 8 col_major combinations (gemm/gemm_baseline.cu:129-168) and K values that are not a multiple of 8 through
    the workspace entry point: operands the kernel cannot read in place are re-packed first."""
    M, N, K = shape
    ac, bc, cc = layout
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0, ac, bc)
    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype, ac, bc, cc)
    need = gpu.matmul_mfma_workspace_bytes(t)
    canonical_in_place = (ac, bc) == (0, 1) and K % 8 == 0
    assert (need == 0) == canonical_in_place
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
    gpu.matmul_mfma_ws(t, ws.data_ptr(), need, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype, ac, bc)
    got = c.cpu().numpy()
    assert H.rel_err(got.T if cc else got, ref) < TOL
    if need:
        with pytest.raises(gpu.MiGemmError):   # too small a workspace is an error, not a silent fallback
            gpu.matmul_mfma_ws(t, ws.data_ptr(), need - 1, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
        with pytest.raises(gpu.MiGemmError):   # and the no-workspace entry point refuses the problem
            gpu.matmul_mfma(t, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())


SUM_SHAPES = [(256, 512, 2048), (300, 500, 1000), (33, 65, 4104), (160, 480, 816), (257, 129, 2040), (1, 1, 640)]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("tile", list(range(14)))
@pytest.mark.parametrize("shape", SUM_SHAPES)
def test_mfma_split_k_workspace_sum(gpu, oracle, dtype, tile, shape):
    """K partitions store private copies of C in the workspace and the copies are summed in partition order, by the
    workgroup that stores a tile's last copy (inside the launch, switched on by hand) or by a second kernel (the default): same accuracy bound as the atomic mode, the same bits on every run and either way, nothing
    stored outside C or the workspace, and an error (not a fallback) when the forced mode gets too little room."""
    M, N, K = shape
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    guard = 4096
    buf = torch.empty(M * N + 2 * guard, dtype=torch.float32, device="cuda")
    c = buf[guard:guard + M * N].view(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype)
    plan = gpu.matmul_mfma_plan(t, gpu.K_SPLIT_REDUCE, tile)
    need, pref = gpu.matmul_mfma_workspace_bytes_for(t, gpu.K_SPLIT_REDUCE, tile)
    assert plan["k_splits"] > 1 and pref == plan["k_splits"] * M * N * 4 and need == 2 * M * N * 4
    ws = torch.empty(pref + 2 * guard * 4, dtype=torch.uint8, device="cuda")
    ws_inner = ws[guard * 4:guard * 4 + pref]
    assert ws_inner.data_ptr() % 256 == 0
    runs = []
    # 0xFF bytes are NaNs: nothing of the old C or workspace may leak into the sum
    for poison, in_launch in ((0x7D, True), (0xFF, True), (0xFF, False)):
        buf.view(torch.uint8).fill_(poison)
        ws.fill_(poison)
        was, calls_before = gpu.matmul_mfma_sum_in_launch(in_launch)
        try:
            gpu.matmul_mfma_ws(t, ws_inner.data_ptr(), pref, gpu.K_SPLIT_REDUCE, tile, H.stream_handle())
            calls = gpu.matmul_mfma_sum_in_launch()[1] - calls_before
        finally:
            gpu.matmul_mfma_sum_in_launch(was)
        torch.cuda.synchronize()
        # (the in-launch sum may fall back when every slab of counters is taken by other workspaces, never the reverse)
        assert calls <= (1 if in_launch else 0)
        runs.append(c.cpu().numpy().copy())
        assert H.rel_err(runs[-1], ref) < TOL, plan
        edges = torch.cat([buf[:guard], buf[guard + M * N:]]).view(torch.uint8)
        assert bool((edges == poison).all()), "stored outside C"
        assert bool((ws[:guard * 4] == poison).all()) and bool((ws[guard * 4 + pref:] == poison).all()), "stored outside the workspace"
    np.testing.assert_array_equal(runs[0], runs[1])
    np.testing.assert_array_equal(runs[0], runs[2])
    # the least room there is: two partitions, still inside the workspace given
    ws.fill_(0x7D)
    c.fill_(float("nan"))
    gpu.matmul_mfma_ws(t, ws_inner.data_ptr(), need, gpu.K_SPLIT_REDUCE, tile, H.stream_handle())
    torch.cuda.synchronize()
    assert H.rel_err(c.cpu().numpy(), ref) < TOL
    assert bool((ws[guard * 4 + need:] == 0x7D).all()), "stored outside the workspace"
    with pytest.raises(gpu.MiGemmError):
        gpu.matmul_mfma_ws(t, ws_inner.data_ptr(), need - 1, gpu.K_SPLIT_REDUCE, tile, H.stream_handle())
    # the partial sums are the atomic mode's addends: the two modes agree to rounding
    gpu.matmul_mfma(t, gpu.K_SPLIT, tile, H.stream_handle())
    torch.cuda.synchronize()
    assert H.rel_err(c.cpu().numpy(), runs[0].astype(np.float64)) < 1e-5


ROTATED_WALK_CASES = [  # (tile name, M, N, K, forced partitions or 0 for the planner's)
    ("TILE_256x256", 256, 256, 32768, 2),    # two workgroups, on XCD 0 (walk from the start) and XCD 1 (37 K tiles in)
    ("TILE_128x128", 512, 512, 32768, 2),    # 32 workgroups: every XCD, the walks of XCD 7 start 3 tiles in (259 mod 256)
    ("TILE_128x128", 512, 512, 32768, 0),
    ("TILE_64x128", 128, 256, 65536, 0),
    ("TILE_256x128", 256, 384, 32768, 0),
]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("case", ROTATED_WALK_CASES)
def test_mfma_split_k_rotated_walk(gpu, oracle, dtype, case):
    """Rows of a power-of-two length of 64 KB or more: the workgroups of XCD x walk their K partition from 37 * x K tiles
    in and wrap around to its start.  Every K tile must still be used exactly once, whatever the partition length."""
    tile_name, M, N, K, forced = case
    tile = getattr(gpu, tile_name)
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 0.5)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype)
    if forced:
        need, _ = gpu.matmul_mfma_workspace_bytes_for(t, gpu.K_SPLIT_REDUCE, tile)
        assert need == forced * M * N * 4
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        gpu.matmul_mfma_ws(t, ws.data_ptr(), need, gpu.K_SPLIT_REDUCE, tile, H.stream_handle())
        k_tiles = K // 64 // forced
    else:
        plan = gpu.matmul_mfma_plan(t, gpu.K_SPLIT, tile)
        assert plan["k_splits"] > 1
        k_tiles = -(-(K // 64) // plan["k_splits"])
        gpu.matmul_mfma(t, gpu.K_SPLIT, tile, H.stream_handle())
    torch.cuda.synchronize()
    assert k_tiles >= 16, "partitions this short are not rotated: the case no longer tests the wrap-around"
    assert H.rel_err(c.cpu().numpy(), ref) < TOL


STREAM_CASES = [  # (tile, bm, bn, tiles_m, tiles_n, K tiles): 4 to 5 K tiles per workgroup; leftover runs cross tiles
    # more tiles than CUs: whole rounds run output stationary, the rest is streamed (272 = 256 + 16 tiles with no
    # leftover workgroups; 280 = 256 + 24 with 16 of them; 552 = 2 * 256 + 40)
    ("TILE_128x128", 128, 128, 17, 16, 64), ("TILE_64x128", 64, 128, 20, 14, 48), ("TILE_64x128", 64, 128, 23, 24, 32),
    ("TILE_256x256", 256, 256, 1, 3, 342), ("TILE_256x256", 256, 256, 3, 1, 343), ("TILE_256x256", 256, 256, 2, 3, 171),
    ("TILE_192x256", 192, 256, 3, 1, 345), ("TILE_256x128", 256, 128, 1, 5, 206), ("TILE_128x128", 128, 128, 3, 3, 115),
    ("TILE_64x128", 64, 128, 5, 2, 103), ("TILE_256x256", 256, 256, 1, 1, 1280), ("TILE_128x128", 128, 128, 7, 9, 18),
    ("TILE_224x256", 224, 256, 3, 1, 343), ("TILE_160x256", 160, 256, 1, 3, 342), ("TILE_224x128", 224, 128, 5, 1, 206),
    ("TILE_160x128", 160, 128, 3, 3, 115), ("TILE_256x192", 256, 192, 1, 3, 342),
    ("TILE_192x192", 192, 192, 3, 2, 171), ("TILE_192x128", 192, 128, 2, 3, 400),
    ("TILE_96x128", 96, 128, 3, 3, 115),
]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("case", STREAM_CASES)
def test_mfma_stream_k(gpu, oracle, dtype, case):
    """Stream-K: whole rounds of tiles output stationary, the tail tiles' K tiles dealt evenly to one round of
    workgroups (main partitions in step, leftover runs across tiles), parts in the workspace, summed in a fixed order by
    the workgroup that stores a tile's last part (switched on by hand) or by a last kernel (the default).  Same bits
    on every run and either way; nothing outside C or the workspace; the forced mode refuses too small a workspace."""
    tile_name, bm, bn, tiles_m, tiles_n, k_tiles = case
    tile = getattr(gpu, tile_name)
    M, N, K = bm * tiles_m, bn * tiles_n, 64 * k_tiles
    a, b = H.make_inputs(M, N, K, dtype, 4, 4, K ** -0.5)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
    guard = 4096
    buf = torch.empty(M * N + 2 * guard, dtype=torch.float32, device="cuda")
    c = buf[guard:guard + M * N].view(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype)
    plan = gpu.matmul_mfma_plan(t, gpu.K_STREAM, tile)
    assert plan["k_mode"] == "stream k"
    need, pref = gpu.matmul_mfma_workspace_bytes_for(t, gpu.K_STREAM, tile)
    assert need == pref and need % (bm * bn * 4) == 0
    ws = torch.empty(need + 2 * guard * 4, dtype=torch.uint8, device="cuda")
    ws_inner = ws[guard * 4:guard * 4 + need]
    runs = []
    for poison, in_launch in ((0x7D, True), (0xFF, True), (0xFF, False)):
        buf.view(torch.uint8).fill_(poison)
        ws.fill_(poison)
        was, _ = gpu.matmul_mfma_sum_in_launch(in_launch)
        try:
            gpu.matmul_mfma_ws(t, ws_inner.data_ptr(), need, gpu.K_STREAM, tile, H.stream_handle())
        finally:
            gpu.matmul_mfma_sum_in_launch(was)
        torch.cuda.synchronize()
        runs.append(c.cpu().numpy().copy())
        assert H.rel_err(runs[-1], ref) < TOL, plan
        edges = torch.cat([buf[:guard], buf[guard + M * N:]]).view(torch.uint8)
        assert bool((edges == poison).all()), "stored outside C"
        assert bool((ws[:guard * 4] == poison).all()) and bool((ws[guard * 4 + need:] == poison).all()), "stored outside the workspace"
    np.testing.assert_array_equal(runs[0], runs[1])
    np.testing.assert_array_equal(runs[0], runs[2])
    with pytest.raises(gpu.MiGemmError):
        gpu.matmul_mfma_ws(t, ws_inner.data_ptr(), need - 1, gpu.K_STREAM, tile, H.stream_handle())


def test_mfma_stream_k_known_answer_and_refusals(gpu, oracle):
    """Identity x tiled numbers is exact whatever the partition of K; ragged shapes, whole rounds of tiles and too
    short a K are refused by the forced mode."""
    M, N, K = 512, 768, 64 * 200
    a, b = H.make_inputs(M, N, K, 0, 1, 2)
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, 0)
    need, _ = gpu.matmul_mfma_workspace_bytes_for(t, gpu.K_STREAM)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    gpu.matmul_mfma_ws(t, ws.data_ptr(), need, gpu.K_STREAM, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    b_logical = oracle.widen(H.to_host_u16(b), 0).T
    np.testing.assert_array_equal(c.cpu().numpy(), b_logical[:M, :])
    for shape in [(500, 768, 12800), (512, 768, 12808), (8192, 8192, 1024), (256, 256, 128)]:
        ts = H.tensors(*shape, a, b, c, 0)
        assert not gpu.matmul_mfma_supports(ts, gpu.K_STREAM, gpu.TILE_AUTO)
        with pytest.raises(gpu.MiGemmError):
            gpu.matmul_mfma_ws(ts, ws.data_ptr(), need, gpu.K_STREAM, gpu.TILE_AUTO, H.stream_handle())


@pytest.mark.parametrize("layout", [(a, b, c) for a in (0, 1) for b in (0, 1) for c in (0, 1)])
def test_mfma_workspace_sum_with_repacked_operands(gpu, oracle, layout):
    """Re-packed operands and the partitions' copies of C share one workspace; every layout, K not a multiple of 8."""
    M, N, K = 150, 77, 2003
    ac, bc, cc = layout
    a, b = H.make_inputs(M, N, K, 1, 3, 3, 1.0, ac, bc)
    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, 1, ac, bc, cc)
    need, pref = gpu.matmul_mfma_workspace_bytes_for(t, gpu.K_SPLIT_REDUCE, gpu.TILE_AUTO)
    assert pref >= need >= gpu.matmul_mfma_workspace_bytes(t) + 2 * M * N * 4
    ws = torch.empty(pref, dtype=torch.uint8, device="cuda")
    ws.fill_(0xFF)
    gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, gpu.K_SPLIT_REDUCE, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), 1, ac, bc)
    got = c.cpu().numpy()
    assert H.rel_err(got.T if cc else got, ref) < TOL


def test_mfma_auto_takes_the_workspace_sum_when_given_room(gpu, oracle):
    """K_AUTO on a deep-K problem: with the preferred workspace the partitions are summed from copies (bitwise
    repeatable), with none they meet through atomics; both within tolerance."""
    M, N, K = 256, 384, 16384
    a, b = H.make_inputs(M, N, K, 1, 4, 4, K ** -0.5)
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), 1)
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, 1)
    req, pref = gpu.matmul_mfma_workspace_bytes_for(t)
    assert req == 0 and pref > 0
    ws = torch.empty(pref, dtype=torch.uint8, device="cuda")
    outs = []
    for _ in range(2):
        c.fill_(float("nan"))
        ws.fill_(0xFF)
        gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
        torch.cuda.synchronize()
        outs.append(c.cpu().numpy().copy())
        assert H.rel_err(outs[-1], ref) < TOL
    np.testing.assert_array_equal(outs[0], outs[1])
    ws.fill_(0x7D)
    gpu.matmul_mfma_ws(t, ws.data_ptr(), 256, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())  # too little room: atomics
    torch.cuda.synchronize()
    assert H.rel_err(c.cpu().numpy(), ref) < TOL
    assert bool((ws == 0x7D).all())


@pytest.mark.parametrize("shape,tile", [((512, 512, 512), "TILE_256x256"), ((1024, 2304, 256), "TILE_64x128"),
                                        ((150, 77, 200), "TILE_AUTO")])
def test_mfma_timeline_entry(gpu, oracle, shape, tile):
    """The diagnostic launch computes the same C and every workgroup leaves ordered stamps: entry, then per work item
    K tile 0 landed, the end of its K loop and of its store issue, then stores landed; the last slot names the CU."""
    M, N, K = shape
    a, b = H.make_inputs(M, N, K, 1, 3, 3, 1.0, 0, 1)
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, 1, 0, 1, 0)
    slots, max_wg = 16, 4096
    stamps = torch.zeros((max_wg, slots, 2), dtype=torch.int64, device="cuda")
    wgs = gpu.matmul_mfma_timeline(t, stamps.data_ptr(), slots, max_wg, gpu.K_OUTPUT_STATIONARY, getattr(gpu, tile),
                                   H.stream_handle())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), 1, 0, 1)
    assert H.rel_err(c.cpu().numpy(), ref) < TOL
    st = stamps.cpu().numpy()
    assert 1 <= wgs <= max_wg
    assert (st[wgs:] == 0).all()
    assert (st[:wgs, slots - 1, 0] != 0).all() and (st[:wgs, slots - 1, 1] < 8).all()   # hardware id + 1, XCC id
    n = (st[:wgs, :slots - 1, 0] != 0).sum(axis=1)
    assert (n >= 5).all() and (n % 3 == 2).all()      # entry + 3 per item + landed
    for g in range(wgs):
        wall = st[g, :n[g], 0]
        core = st[g, :n[g], 1]
        assert (wall[1:] >= wall[:-1]).all() and (core[1:] > core[:-1]).all()
    # a buffer too small for the grid is refused before anything is launched
    with pytest.raises(gpu.MiGemmError):
        gpu.matmul_mfma_timeline(t, stamps.data_ptr(), slots, 0 if wgs == 1 else wgs - 1, gpu.K_OUTPUT_STATIONARY,
                                 getattr(gpu, tile), H.stream_handle())


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("layout", [(0, 1, 0), (0, 0, 0), (1, 1, 0), (1, 0, 1), (0, 1, 1)])
def test_vendor_comparator_agrees_with_the_oracle(gpu, oracle, dtype, layout):
    """The hipBLASLt row computes the same product from the same buffers (so that timing it beside the MFMA kernel
    compares like with like): fp32 output, every layout flag."""
    from spork_amd import vendor as V

    if not V.enabled():
        pytest.skip("hipBLASLt handle could not be created")
    M, N, K = 384, 256, 512
    ac, bc, cc = layout
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0, ac, bc)
    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype, ac, bc, cc)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    V.matmul(t, ws.data_ptr(), ws.numel(), H.stream_handle())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype, ac, bc)
    got = c.cpu().numpy()
    assert H.rel_err(got.T if cc else got, ref) < TOL


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("case", [
    # (M, N, K), batches, c_col_major, k_mode, tile, pad elements between problems (A, B, C)
    ((256, 384, 512), 3, 0, "K_OUTPUT_STATIONARY", "TILE_128x128", (0, 0, 0)),
    ((256, 384, 512), 3, 1, "K_AUTO", "TILE_AUTO", (0, 0, 0)),          # C[L,N,M]: the reference's batched layout
    ((200, 136, 264), 4, 0, "K_AUTO", "TILE_AUTO", (64, 128, 36)),      # ragged shape, strided batches
    ((256, 256, 1024), 2, 0, "K_SPLIT", "TILE_256x256", (0, 0, 4096)),  # split K: every problem's C is zero-filled
])
def test_mfma_batched(gpu, oracle, dtype, case):
    """L problems of one shape in one launch (the leading `L` of xgemm_Sm90_wgmma, xgemm_Sm90.py:43-48): each problem
    equals the oracle's product of its own slices, nothing is written between the problems' C matrices, and with the
    tile fixed the result is bit-identical to L separate calls."""
    (M, N, K), L, cc, k_mode, tile, (pad_a, pad_b, pad_c) = case
    sa, sb, sc = M * K + pad_a, N * K + pad_b, M * N + pad_c
    a = torch.empty(L * sa, dtype=torch.int16, device="cuda")
    b = torch.empty(L * sb, dtype=torch.int16, device="cuda")
    c = torch.empty(L * sc, dtype=torch.float32, device="cuda")
    c.view(torch.uint8).fill_(0x7D)
    st = H.stream_handle()
    for l in range(L):
        gpu.init_test_data(a[l * sa:].data_ptr(), M, K, 3, False, dtype, 1.0, 1000 + l, st)
        gpu.init_test_data(b[l * sb:].data_ptr(), N, K, 3, True, dtype, 1.0, 2000 + l, st)
    t = gpu.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), dtype, 0, 1, cc)
    strides = (0, 0, 0) if (pad_a, pad_b, pad_c) == (0, 0, 0) else (sa, sb, sc)
    gpu.matmul_mfma_batched(t, L, *strides, getattr(gpu, k_mode), getattr(gpu, tile), st)
    torch.cuda.synchronize()
    ha, hb, hc = a.cpu().numpy().view("uint16"), b.cpu().numpy().view("uint16"), c.cpu().numpy()
    poison = hc.view("uint32")
    for l in range(L):
        ref = oracle.gemm_f64(M, N, K, ha[l * sa:l * sa + M * K].reshape(M, K), hb[l * sb:l * sb + N * K].reshape(N, K), dtype)
        got = hc[l * sc:l * sc + M * N].reshape((N, M) if cc else (M, N))
        assert H.rel_err(got.T if cc else got, ref) < TOL, l
        assert (poison[l * sc + M * N:(l + 1) * sc] == 0x7D7D7D7D).all(), l   # the gap after problem l is untouched
    if k_mode == "K_OUTPUT_STATIONARY":
        for l in range(L):
            c1 = H.poisoned_c(M, N)
            t1 = gpu.GpuTensors.make(M, N, K, a[l * sa:].data_ptr(), b[l * sb:].data_ptr(), c1.data_ptr(), dtype, 0, 1, cc)
            gpu.matmul_mfma(t1, getattr(gpu, k_mode), getattr(gpu, tile), st)
            torch.cuda.synchronize()
            assert (c1.cpu().numpy().ravel() == hc[l * sc:l * sc + M * N]).all()


@pytest.mark.parametrize("precision,tol", [("F32_BF16X3", 3e-5), ("F32_BF16X1", 1e-2)])
@pytest.mark.parametrize("layout", [(0, 1, 0), (0, 0, 0), (1, 0, 1), (1, 1, 0)])
@pytest.mark.parametrize("shape", [(300, 200, 100), (512, 256, 768)])
def test_f32_inputs(gpu, precision, tol, layout, shape):
    """fp32 A and B (the reference's element type, gemm/gpu_tensor.h:14-16) through the bf16 split: against numpy's
    float64 product of the same fp32 values.  Three terms carry 16 significant bits per operand (TF32 carries 11),
    one term 8."""
    import numpy as np

    M, N, K = shape
    ac, bc, cc = layout
    g = torch.Generator(device="cuda").manual_seed(1234)
    a_log = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32)       # logical A[m,k]
    b_log = torch.randn((K, N), generator=g, device="cuda", dtype=torch.float32)       # logical B[k,n]
    a = a_log.t().contiguous() if ac else a_log.contiguous()                           # col-major A is stored K x M
    b = b_log.t().contiguous() if bc else b_log.contiguous()                           # col-major B is stored N x K
    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    t = gpu.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), gpu.F32, ac, bc, cc)
    prec = getattr(gpu, precision)
    need = gpu.matmul_f32_workspace_bytes(t, prec)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    gpu.matmul_f32_ws(t, ws.data_ptr(), need, prec, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    ref = a_log.cpu().numpy().astype(np.float64) @ b_log.cpu().numpy().astype(np.float64)
    got = c.cpu().numpy()
    assert H.rel_err(got.T if cc else got, ref) < tol
    with pytest.raises(gpu.MiGemmError):
        gpu.matmul_f32_ws(t, ws.data_ptr(), need - 1, prec, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())


def test_f32_inputs_conversion_paths_agree(gpu):
    """The conversion has a 16-byte path for aligned K-contiguous rows with K % 8 == 0 and an element-wise one for the
    rest: the same A and B, once aligned and once starting 4 bytes into their buffers, give the same bits."""
    M, N, K = 328, 200, 776
    g = torch.Generator(device="cuda").manual_seed(4321)
    a_buf = torch.randn(M * K + 4, generator=g, device="cuda", dtype=torch.float32)
    b_buf = torch.randn(N * K + 4, generator=g, device="cuda", dtype=torch.float32)
    a_off, b_off = a_buf[1:1 + M * K], b_buf[1:1 + N * K]          # 4 bytes past a 16-byte boundary
    a_al, b_al = a_off.clone(), b_off.clone()
    assert a_al.data_ptr() % 16 == 0 and a_off.data_ptr() % 16 == 4
    out = []
    for a, b in ((a_al, b_al), (a_off, b_off)):
        c = H.poisoned_c(M, N)
        t = gpu.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), gpu.F32, 0, 1, 0)
        need = gpu.matmul_f32_workspace_bytes(t, gpu.F32_BF16X3)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        gpu.matmul_f32_ws(t, ws.data_ptr(), need, gpu.F32_BF16X3, gpu.K_OUTPUT_STATIONARY, gpu.TILE_128x128, H.stream_handle())
        torch.cuda.synchronize()
        out.append(c)
    assert torch.equal(out[0], out[1])


def test_f32_inputs_known_answer(gpu):
    """The reference's own known answer in its own element type (gemm/gemm_main.cpp:81-90, gemm/gemm_test.cu:67-72):
    tiled numbers up to 6363 times the identity.  Two bf16 terms hold every integer below 65536 exactly, so the
    three-term product returns A bit for bit; one term returns A rounded to bf16."""
    import numpy as np

    M = N = K = 384
    yy, xx = np.meshgrid(np.arange(M), np.arange(K), indexing="ij")
    a_host = ((xx % 64) + 100 * (yy % 64)).astype(np.float32)
    assert a_host.max() == 6363
    a = torch.from_numpy(a_host).cuda()
    b = torch.eye(N, K, dtype=torch.float32, device="cuda")
    for prec in (gpu.F32_BF16X3, gpu.F32_BF16X1):
        c = H.poisoned_c(M, N)
        t = gpu.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), gpu.F32, 0, 1, 0)
        need = gpu.matmul_f32_workspace_bytes(t, prec)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        gpu.matmul_f32_ws(t, ws.data_ptr(), need, prec, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
        torch.cuda.synchronize()
        want = a if prec == gpu.F32_BF16X3 else a.to(torch.bfloat16).to(torch.float32)
        assert torch.equal(c, want)


def _xgemm_ctxt(gpu, L, M, N, K, precision, tile=0, slack=0):
    need = gpu.xgemm_workspace_bytes(L, M, N, K, precision)
    ws = torch.empty(need + slack, dtype=torch.uint8, device="cuda")
    return gpu.XgemmContext(ws.data_ptr(), need + slack, H.stream_handle(), precision, tile), ws


@pytest.mark.parametrize("precision,tol", [("F32_BF16X3", 3e-5), ("F32_BF16X1", 1e-2)])
@pytest.mark.parametrize("shape", [(192, 256, 64), (384, 512, 1024), (300, 200, 100)])
def test_xgemm_sm80_argument_list(gpu, precision, tol, shape):
    """xgemm_Sm80_fence(ctxt, M, N, K, A f32[M,K], B f32[K,N], C f32[M,N]) (xgemm_Sm80.py:18-21, called at
    gemm/gemm_test.cu:326): against numpy's float64 product, on the proc's smallest legal shape (one 192 x 256 tile,
    K % 16), a multiple of it, and a shape its assertions exclude but the interface admits."""
    import numpy as np

    M, N, K = shape
    g = torch.Generator(device="cuda").manual_seed(80)
    a = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32)
    b = torch.randn((K, N), generator=g, device="cuda", dtype=torch.float32)
    c = H.poisoned_c(M, N)
    ctxt, _ws = _xgemm_ctxt(gpu, 1, M, N, K, getattr(gpu, precision))
    gpu.xgemm_Sm80(ctxt, M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    ref = a.cpu().numpy().astype(np.float64) @ b.cpu().numpy().astype(np.float64)
    assert H.rel_err(c.cpu().numpy(), ref) < tol


@pytest.mark.parametrize("case", [
    # L, M, N, K_splits, cluster_k, tile
    (2, 500, 800, 1, 240, "TILE_AUTO"),      # the reference's own check of the proc (xgemm_Sm90.py:203)
    (2, 500, 800, 2, 240, "TILE_AUTO"),      # ... and of its split-K build (:202)
    (1, 512, 384, 1, 1024, "TILE_256x256"),  # L = 1, as the harness calls it (gemm/gemm_test.cu:335)
    (1, 256, 256, 8, 512, "TILE_128x128"),   # the harness's K splits (gemm/gemm_test.cu:341-355)
    (5, 64, 72, 1, 36, "TILE_AUTO"),         # many small ragged problems in one launch
    (3, 200, 136, 4, 68, "TILE_64x128"),     # split K zero-fills every problem's C
])
def test_xgemm_sm90_argument_list(gpu, case):
    """xgemm_Sm90_wgmma(ctxt, L, M, N, K_splits, cluster_k, A f32[L,M,K], B f32[L,N,K], C f32[L,N,M])
    (xgemm_Sm90.py:43-48): every problem against numpy's float64 product of its own slices; C arrives poisoned, so the
    split-K cases also show that the entry zero-fills before the partitions add (xgemm_Sm90.py:60-61)."""
    import numpy as np

    L, M, N, K_splits, cluster_k, tile = case
    K = K_splits * cluster_k
    g = torch.Generator(device="cuda").manual_seed(90)
    a = torch.randn((L, M, K), generator=g, device="cuda", dtype=torch.float32)
    b = torch.randn((L, N, K), generator=g, device="cuda", dtype=torch.float32)
    c = torch.empty((L, N, M), dtype=torch.float32, device="cuda")
    c.view(torch.uint8).fill_(0x7D)
    ctxt, _ws = _xgemm_ctxt(gpu, L, M, N, K, gpu.F32_BF16X3, getattr(gpu, tile))
    gpu.xgemm_Sm90_wgmma(ctxt, L, M, N, K_splits, cluster_k, a.data_ptr(), b.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    ha, hb, hc = a.cpu().numpy().astype(np.float64), b.cpu().numpy().astype(np.float64), c.cpu().numpy()
    for l in range(L):
        assert H.rel_err(hc[l], hb[l] @ ha[l].T) < 3e-5, l


def test_xgemm_sm90_as_the_harness_calls_it(gpu, oracle):
    """The reference's harness passes (1, N, M, 1, K, B column-major, A, C) - operands swapped - so that C[L,N,M] is its
    row-major M x N (gemm/gemm_test.cu:335).  The same call here on 16-bit test data widened to fp32 gives what the
    16-bit entry point gives on the data itself, to fp32 rounding: bf16 values split into (value, 0) exactly."""
    M, N, K = 320, 448, 512
    dtype = gpu.BF16
    a16 = H.gen_on_device(M, K, 3, False, dtype, 1.0, 1)
    b16 = H.gen_on_device(N, K, 3, True, dtype, 1.0, 2)
    a32 = torch.empty((M, K), dtype=torch.float32, device="cuda")
    b32 = torch.empty((N, K), dtype=torch.float32, device="cuda")
    st = H.stream_handle()
    gpu.widen_to_f32(a16.data_ptr(), dtype, a32.data_ptr(), M * K, st)
    gpu.widen_to_f32(b16.data_ptr(), dtype, b32.data_ptr(), N * K, st)
    torch.cuda.synchronize()
    assert torch.equal(a32, a16.view(torch.bfloat16).to(torch.float32).reshape(M, K))
    c = H.poisoned_c(M, N)
    ctxt, _ws = _xgemm_ctxt(gpu, 1, N, M, K, gpu.F32_BF16X3)
    gpu.xgemm_Sm90_wgmma(ctxt, 1, N, M, 1, K, b32.data_ptr(), a32.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(M, N, K, a16.cpu().numpy().view("uint16").reshape(M, K), b16.cpu().numpy().view("uint16").reshape(N, K), dtype)
    assert H.rel_err(c.cpu().numpy(), ref) < 1e-5


def test_xgemm_null_context_is_the_reference_call_form(gpu):
    """The harness line verbatim, `xgemm_Sm90_wgmma_n256(nullptr, 1, N, M, 1, K, d_bCol, d_a, d_c)` on stream 0
    (gemm/gemm_test.cu:335), and `xgemm_Sm80_fence(nullptr, M, N, K, d_a, d_b, d_c)` (:326): a null context means stream 0,
    bf16x3 and the library's resident scratch array.  1024^3 (12 MiB of converted operands) against numpy's float64
    product, twice in a row with a smaller problem second (the array keeps the last call's bytes); 8192^3 (768 MiB) is
    refused with MI_ERR_WORKSPACE and leaves C alone."""
    import ctypes as C

    import numpy as np

    lib = gpu.lib()
    g = torch.Generator(device="cuda").manual_seed(335)
    for M, N, K in ((1024, 1024, 1024), (320, 200, 136)):
        a = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32)
        b_col = torch.randn((N, K), generator=g, device="cuda", dtype=torch.float32)   # B stored N x K: the harness's d_bCol
        c = H.poisoned_c(M, N)
        torch.cuda.synchronize()
        gpu.xgemm_Sm90_wgmma(None, 1, N, M, 1, K, b_col.data_ptr(), a.data_ptr(), c.data_ptr())
        torch.cuda.synchronize()
        ha, hb = a.cpu().numpy().astype(np.float64), b_col.cpu().numpy().astype(np.float64)
        assert H.rel_err(c.cpu().numpy(), ha @ hb.T) < 3e-5, (M, N, K)
        b_rows = b_col.t().contiguous()                                               # K x N row-major: the harness's d_b
        c2 = H.poisoned_c(M, N)
        torch.cuda.synchronize()
        gpu.xgemm_Sm80(None, M, N, K, a.data_ptr(), b_rows.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        assert H.rel_err(c2.cpu().numpy(), ha @ hb.T) < 3e-5, (M, N, K)
    big = 8192
    assert gpu.xgemm_workspace_bytes(1, big, big, big) > gpu.STATIC_SCRATCH_BYTES
    before = c.clone()
    p = c.data_ptr()  # (refused before any operand is touched: the addresses only have to be non-null)
    assert lib.mi_xgemm_Sm90_wgmma(None, 1, big, big, 1, big, p, p, p) == 3
    assert lib.mi_xgemm_Sm80(None, big, big, big, p, p, p) == 3
    torch.cuda.synchronize()
    assert torch.equal(c, before)


@pytest.mark.parametrize("tile", [16, 32])
def test_mfma_ceiling_probe(gpu, tile):
    """The MFMA-only measurement loop runs on every CU, reports plausible clocks and the flop it performed; on zeros
    it issues back to back (16 or 32 cycles per instruction)."""
    import ctypes as C

    lib = gpu.lib()
    ops = torch.zeros(32 << 20, dtype=torch.uint8, device="cuda")
    clocks = torch.zeros(2 * 1024, dtype=torch.int64, device="cuda")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    wgs, flop = C.c_uint32(), C.c_double()
    iters = 200
    st = lib.mi_mfma_ceiling(ops.data_ptr(), ops.numel(), gpu.BF16, tile, iters, clocks.data_ptr(), sink.data_ptr(),
                             C.byref(wgs), C.byref(flop), H.stream_handle())
    assert st == 0
    torch.cuda.synchronize()
    assert wgs.value >= 1
    per_iter = 2 * (16 * 32768 if tile == 32 else 64 * 16384)
    assert flop.value == wgs.value * 4 * iters * per_iter
    h = clocks.cpu().numpy()[: 2 * wgs.value].reshape(-1, 2)
    assert (h > 0).all() and (clocks.cpu().numpy()[2 * wgs.value:] == 0).all()
    mfmas = iters * 2 * (16 if tile == 32 else 64)
    cycles_per_mfma = h[:, 0].mean() / mfmas
    assert 0.95 * (32 if tile == 32 else 16) < cycles_per_mfma < 1.3 * (32 if tile == 32 else 16)
    too_small = lib.mi_mfma_ceiling(ops.data_ptr(), 1024, gpu.BF16, tile, iters, clocks.data_ptr(), sink.data_ptr(),
                                    C.byref(wgs), C.byref(flop), H.stream_handle())
    assert too_small == 3


def test_streaming_probes(gpu):
    """The memory-streaming probes run in every mode and move what they say: the copy copies, the read-only modes leave
    the source alone and take a plausible time (well over 1 TB/s on 64 MB), and a buffer that is not a whole number of
    pieces is covered up to its last whole piece."""
    n = 64 << 20
    src = torch.randint(0, 255, (n + 1024,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    st = H.stream_handle()
    before = src.clone()

    def timed_us(launch):
        for _ in range(3):
            launch()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            launch()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / 5

    gpu.hbm_stream_ceiling(src.data_ptr(), dst.data_ptr(), n + 16, gpu.STREAM_COPY, 4, sink.data_ptr(), st)
    torch.cuda.synchronize()
    assert torch.equal(dst[:n + 16], src[:n + 16]) and not bool(dst[n + 16:].any())
    for mode, per_cu in ((gpu.STREAM_READ, 1), (gpu.STREAM_READ, 8), (gpu.STREAM_DMA, 1), (gpu.STREAM_DMA, 2)):
        us = timed_us(lambda: gpu.hbm_stream_ceiling(src.data_ptr(), 0, n + 512, mode, per_cu, sink.data_ptr(), st))
        assert n / us * 1e-6 > 1.0, (mode, per_cu, us)
    for rows_per_wg in (8, 64, 128):
        us = timed_us(lambda: gpu.hbm_stream_rows_ceiling(src.data_ptr(), 4096, 16384, rows_per_wg, st))
        assert n / us * 1e-6 > 1.0, (rows_per_wg, us)
    assert torch.equal(src, before)


@pytest.mark.parametrize("name,dtype", [("f16", 0), ("bf16", 1)])
@pytest.mark.parametrize("layout", [(a, b, c) for a in (0, 1) for b in (0, 1) for c in (0, 1)])
def test_against_the_committed_golden_fixture(gpu, name, dtype, layout):
    """The committed fixture (tests/golden/gemm_small.npz: 48x40x80 operand bit patterns in both storage orders and
    numpy's float64 product, written without the oracle): the MFMA path and the baseline kernel both
    reproduce it from the fixture's own bytes, in all 8 layout combinations."""
    import os

    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemm_small.npz"))
    M, N, K = 48, 40, 80
    ac, bc, cc = layout
    a = H.to_dev_u16(g[f"{name}_a_{'colmajor' if ac else 'rowmajor'}"])
    b = H.to_dev_u16(g[f"{name}_b_{'colmajor' if bc else 'rowmajor'}"])
    want = g[f"{name}_c_f64"]
    st = H.stream_handle()

    def check(c):
        torch.cuda.synchronize()
        got = c.cpu().numpy()
        assert H.rel_err(got.T if cc else got, want) < TOL

    c = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, dtype, ac, bc, cc)
    need = gpu.matmul_mfma_workspace_bytes(t)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
    gpu.matmul_mfma_ws(t, ws.data_ptr(), need, gpu.K_AUTO, gpu.TILE_AUTO, st)
    check(c)
    c2 = H.poisoned_c(N, M) if cc else H.poisoned_c(M, N)
    gpu.matmul_baseline(H.tensors(M, N, K, a, b, c2, dtype, ac, bc, cc), st)
    check(c2)


def test_mfma_rejects_unsupported(gpu):
    a = H.dev_u16(100, 100)
    c = H.poisoned_c(100, 100)
    t = H.tensors(100, 100, 100, a, a, c, 0)
    assert not gpu.matmul_mfma_supports(t)
    with pytest.raises(gpu.MiGemmError):
        gpu.matmul_mfma(t)
    t = H.tensors(256, 256, 256, a, a, c, 0, a_col_major=1)  # A not K-contiguous
    assert not gpu.matmul_mfma_supports(t)


def test_compare_tensors_matches_reference_rule(gpu, oracle):
    rng = np.random.default_rng(5)
    x = rng.random((64, 100), dtype=np.float32)
    y = x.copy()
    y[10, 7] *= 1.05   # ratio failure
    y[3, 90] = -y[3, 90]  # sign failure (earlier in row-major order)
    y[40, 2] *= 1.02   # within 1/32: passes
    dx, dy = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    res = torch.zeros(4, dtype=torch.int64, device="cuda")
    gpu.compare_tensors(dx.data_ptr(), dy.data_ptr(), 64, 100, res.data_ptr(), H.stream_handle())
    torch.cuda.synchronize()
    r = res.cpu().numpy().view(np.uint64)
    assert oracle.compare_ratio(x, y) == (3, 90)
    assert (int(r[0]) >> 32, int(r[0]) & 0xFFFFFFFF) == (3, 90)
    assert int(r[3]) == 2
    assert np.array([r[1]]).view(np.float64)[0] == np.abs(x.astype(np.float64) - y.astype(np.float64)).max()
    assert np.array([r[2]]).view(np.float64)[0] == np.abs(x).max()


def test_host_threads_on_streams_of_their_own(gpu, oracle):
    """Four host threads, each with its own stream and buffers, launch different problems at the same time (the calls
    release the interpreter lock): every thread's results equal what one thread computes alone.  The library keeps no
    state between calls apart from per-device flags, so callers need no lock of their own.  (The exception, not exercised
    here: the entry points that work in the library's one scratch array per GPU - mi_matmul_mfma_static and the Exo entry
    points with a null context - share that array, and calls of those that overlap in time on one GPU must be serialised
    by the caller; each thread below brings a workspace of its own.)"""
    import threading

    problems = [(512, 384, 1024, 0, "K_AUTO"), (300, 200, 1000, 1, "K_AUTO"), (256, 256, 4096, 0, "K_SPLIT_REDUCE"),
                (1024, 128, 2048, 1, "K_OUTPUT_STATIONARY")]
    setups = []
    for M, N, K, dtype, k_mode in problems:
        a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0)
        c_alone, c_threaded = H.poisoned_c(M, N), H.poisoned_c(M, N)
        t_alone, t_threaded = H.tensors(M, N, K, a, b, c_alone, dtype), H.tensors(M, N, K, a, b, c_threaded, dtype)
        _, pref = gpu.matmul_mfma_workspace_bytes_for(t_alone, getattr(gpu, k_mode), gpu.TILE_AUTO)
        ws = torch.empty(max(pref, 256), dtype=torch.uint8, device="cuda")
        gpu.matmul_mfma_ws(t_alone, ws.data_ptr(), pref, getattr(gpu, k_mode), gpu.TILE_AUTO, H.stream_handle())
        setups.append((t_threaded, ws, pref, getattr(gpu, k_mode), c_alone, c_threaded, a, b))
    torch.cuda.synchronize()
    errors = []

    def worker(setup):
        try:
            t, ws, pref, k_mode, _, c_threaded, _, _ = setup
            stream = torch.cuda.Stream()
            for _ in range(50):
                gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, k_mode, gpu.TILE_AUTO, stream.cuda_stream)
            stream.synchronize()
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(s,)) for s in setups]
    for th in threads:
        th.start()
    for th in threads:
        th.join(60)
    assert not errors and not any(th.is_alive() for th in threads), errors
    torch.cuda.synchronize()
    for (t, ws, pref, k_mode, c_alone, c_threaded, a, b), (M, N, K, dtype, _) in zip(setups, problems):
        assert torch.equal(c_alone, c_threaded), (M, N, K)
        ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype)
        assert H.rel_err(c_threaded.cpu().numpy(), ref) < TOL
