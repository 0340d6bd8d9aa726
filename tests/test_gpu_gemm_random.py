"""Seeded random differential test: random shapes, layouts, dtypes, K modes, tiles and workspace sizes through the C
ABI against the on-device baseline kernel (itself pinned against the oracle elsewhere).  C and the workspace sit inside
poisoned guard bands so that a store outside either is caught; C starts as NaN so that an element never written is too."""
import os
import random

import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

TOL = 1e-3


def _cases(seed, count, big):
    rng = random.Random(seed)
    out = []
    for _ in range(count):
        if big:
            # a little over or under a multiple of the large tiles: the in-between tiles, re-packing and now and then
            # peeling are taken (peeling has its own test in test_gpu_gemm_configs.py)
            M = rng.choice([2048, 4096, 6144, 8192]) + rng.choice([-8, 0, 4, 8, 16, 40])
            N = rng.choice([1536, 2048, 4096, 6144]) + rng.choice([-8, 0, 4, 8, 12, 48])
            K = rng.choice([1024, 2048, 4096]) + rng.choice([0, 0, 0, 8, 72])
        else:
            M = rng.choice([rng.randrange(1, 64), rng.randrange(64, 700), rng.choice([128, 256, 512])])
            N = rng.choice([rng.randrange(1, 64), rng.randrange(64, 700), rng.choice([128, 256, 384])])
            K = rng.choice([rng.randrange(1, 40), rng.randrange(8, 3000), 8 * rng.randrange(1, 300), 64 * rng.randrange(1, 40)])
        modes = ["K_AUTO", "K_AUTO", "K_OUTPUT_STATIONARY"] + ([] if big else ["K_SPLIT", "K_SPLIT_REDUCE", "K_STREAM"])
        tiles = [0, 0, 0] + ([rng.randrange(1, 14)] if big else list(range(1, 14)))
        out.append((M, N, K, rng.randrange(2), rng.randrange(2), rng.randrange(2), rng.randrange(2), rng.choice(modes),
                    rng.choice(tiles), rng.choice(["none", "required", "preferred", "between", "huge"])))
    return out


def _run_case(gpu, case):
    M, N, K, dtype, ac, bc, cc, k_mode_name, tile, ws_kind = case
    k_mode = getattr(gpu, k_mode_name)
    a, b = H.make_inputs(M, N, K, dtype, 4, 4, K ** -0.5, ac, bc)
    guard = 2048
    rows, cols = (N, M) if cc else (M, N)
    buf = torch.full((rows * cols + 2 * guard,), float("nan"), dtype=torch.float32, device="cuda")
    c = buf[guard:guard + rows * cols].view(rows, cols)
    t = H.tensors(M, N, K, a, b, c, dtype, ac, bc, cc)
    try:
        required, preferred = gpu.matmul_mfma_workspace_bytes_for(t, k_mode, tile)
    except gpu.MiGemmError:
        return "unsupported"           # e.g. stream-K on a ragged shape: the library says so, nothing runs
    size = {"none": 0, "required": required, "preferred": preferred, "between": (required + preferred) // 2 // 256 * 256,
            "huge": preferred + (8 << 20)}[ws_kind]
    if size < required:
        if required and ws_kind == "none":
            with pytest.raises(gpu.MiGemmError):
                gpu.matmul_mfma(t, k_mode, tile, H.stream_handle())
        return "needs workspace"
    wsbuf = torch.full((size + 2 * guard * 4,), 0xA5, dtype=torch.uint8, device="cuda")
    ws = wsbuf[guard * 4:guard * 4 + size]
    if size == 0:
        if k_mode in (gpu.K_SPLIT_REDUCE, gpu.K_STREAM) and gpu.matmul_mfma_plan(t, k_mode, tile)["k_mode_code"] == k_mode:
            return "needs workspace"
        gpu.matmul_mfma(t, k_mode, tile, H.stream_handle())
    else:
        # (about half of the cases sum their K partitions or stream-K parts inside the GEMM launch, the rest by a launch
        # of its own, which is the library's default)
        was, _ = gpu.matmul_mfma_sum_in_launch((M + N + K // 8) % 2)
        try:
            gpu.matmul_mfma_ws(t, ws.data_ptr(), size, k_mode, tile, H.stream_handle())
        finally:
            gpu.matmul_mfma_sum_in_launch(was)
    ref = torch.empty((M, N), dtype=torch.float32, device="cuda")
    gpu.matmul_baseline(H.tensors(M, N, K, a, b, ref, dtype, ac, bc, 0), H.stream_handle())
    torch.cuda.synchronize()
    what = gpu.matmul_mfma_describe(t, k_mode, tile, size)
    assert bool(torch.isnan(buf[:guard]).all()) and bool(torch.isnan(buf[guard + rows * cols:]).all()), ("stored outside C", case, what)
    assert bool((wsbuf[:guard * 4] == 0xA5).all()) and bool((wsbuf[guard * 4 + size:] == 0xA5).all()), ("stored outside the workspace", case, what)
    got = c.t() if cc else c
    assert not bool(torch.isnan(got).any()), ("element of C never written", case, what)
    scale = float(ref.abs().max())
    err = float((got - ref).abs().max()) / max(scale, 1e-30)
    assert err < TOL, (case, what, err)
    return what


# MI_GEMM_FUZZ_SEEDS=n widens the sweep to n seeds of each kind (120 small or 24 large cases per seed; a few thousand small
# cases take seconds)
_SEEDS = int(os.environ.get("MI_GEMM_FUZZ_SEEDS", "0"))


@pytest.mark.parametrize("seed", list(range(1, max(_SEEDS, 20) + 1)))
def test_random_small_problems_against_the_device_baseline(gpu, seed):
    ran = 0
    for case in _cases(seed, 120, big=False):
        ran += _run_case(gpu, case) not in ("unsupported", "needs workspace")
    assert ran >= 60


@pytest.mark.parametrize("seed", list(range(7, 7 + max(_SEEDS, 4))))
def test_random_large_ragged_problems_against_the_device_baseline(gpu, seed):
    plans = [_run_case(gpu, case) for case in _cases(seed, 24, big=True)]
    assert sum(p not in ("unsupported", "needs workspace") for p in plans) >= 12


def _xgemm_cases(seed, count):
    rng = random.Random(seed)
    out = []
    for _ in range(count):
        k_splits = rng.choice([1, 1, 2, 3, 5])
        cluster_k = rng.choice([rng.randint(1, 300), 8 * rng.randint(1, 60)])
        out.append((rng.choice([1, 1, 2, 3, 7]), rng.randint(1, 700), rng.randint(1, 700), k_splits, cluster_k,
                    rng.choice(["F32_BF16X3", "F32_BF16X3", "F32_BF16X1"])))
    return out


@pytest.mark.parametrize("case", _xgemm_cases(7, 40), ids=lambda c: "L%dx%dx%dx(%dx%d)_%s" % c)
def test_random_xgemm_argument_lists(gpu, case):
    """Random shapes (any M, N, cluster_k; L problems; K splits) through the entry points with the reference's Exo
    argument lists (xgemm_Sm90.py:43-48, xgemm_Sm80.py:18-21) against numpy's float64 product of the same fp32 values; C
    starts as NaN and the workspace ends in a poisoned band."""
    L, M, N, k_splits, cluster_k, precision = case
    K = k_splits * cluster_k
    prec = getattr(gpu, precision)
    tol = 3e-5 if precision == "F32_BF16X3" else 1.5e-2
    g = torch.Generator(device="cuda").manual_seed(L * 1000003 + M * 1009 + N * 13 + K)
    a = torch.randn((L, M, K), generator=g, device="cuda", dtype=torch.float32)
    b = torch.randn((L, N, K), generator=g, device="cuda", dtype=torch.float32)
    c = torch.full((L, N, M), float("nan"), dtype=torch.float32, device="cuda")
    need = gpu.xgemm_workspace_bytes(L, M, N, K, prec)
    ws = torch.full((need + 512,), 0xAB, dtype=torch.uint8, device="cuda")
    ctxt = gpu.XgemmContext(ws.data_ptr(), need, H.stream_handle(), prec, gpu.TILE_AUTO)
    gpu.xgemm_Sm90_wgmma(ctxt, L, M, N, k_splits, cluster_k, a.data_ptr(), b.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    assert bool((ws[need:] == 0xAB).all()), "wrote past the workspace"
    ref = np.einsum("lnk,lmk->lnm", b.cpu().numpy().astype(np.float64), a.cpu().numpy().astype(np.float64))
    scale = max(np.abs(ref).max(), 1e-300)
    assert np.nanmax(np.abs(c.cpu().numpy() - ref)) / scale < tol and not torch.isnan(c).any()
    if L == 1:
        b_rows = b[0].t().contiguous()  # K x N, as the Sm80 proc takes it
        c2 = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        gpu.xgemm_Sm80(ctxt, M, N, K, a.data_ptr(), b_rows.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        assert bool((ws[need:] == 0xAB).all()), "wrote past the workspace"
        assert np.nanmax(np.abs(c2.cpu().numpy() - ref[0].T)) / scale < tol and not torch.isnan(c2).any()
