"""Every GEMM entry point issues kernels only (zero fills are kernels, not memset nodes), so a caller may capture a
call into a HIP graph.  Each case is captured once and replayed several times on inputs that change between replays,
with eager work and synchronisation in between; every replay is compared with an eager call on the same inputs."""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

CASES = {
    # name: (M, N, K, k_mode, tile, uses workspace)
    "output_stationary": (512, 768, 1024, "K_OUTPUT_STATIONARY", "TILE_256x256", False),
    "split_k_atomics": (256, 384, 4096, "K_SPLIT", "TILE_128x128", False),      # fill kernel + atomic kernel
    "split_k_workspace_sum": (256, 384, 4096, "K_SPLIT_REDUCE", "TILE_128x128", True),
    "stream_k": (512, 768, 64 * 171, "K_STREAM", "TILE_256x256", True),
    "ragged_edge_build": (300, 500, 1000, "K_AUTO", "TILE_AUTO", False),
    "peeled": (1028, 4096, 4096, "K_AUTO", "TILE_AUTO", False),                 # three launches, one with a 2-D fill
    "repacked_operands": (150, 77, 203, "K_AUTO", "TILE_AUTO", True),           # re-pack kernels, then the GEMM
}


@pytest.mark.parametrize("name", list(CASES))
def test_entry_points_replay_correctly_from_a_graph(gpu, name):
    M, N, K, k_mode, tile, with_ws = CASES[name]
    k_mode, tile = getattr(gpu, k_mode), getattr(gpu, tile)
    repack = name == "repacked_operands"
    dtype = 1
    a = H.dev_u16(K, M) if repack else H.dev_u16(M, K)       # column-major A for the re-pack case
    b = H.dev_u16(K, N) if repack else H.dev_u16(N, K)       # row-major B for the re-pack case
    c_graph, c_eager = H.poisoned_c(M, N), H.poisoned_c(M, N)
    flags = (1, 0, 0) if repack else (0, 1, 0)
    tg = H.tensors(M, N, K, a, b, c_graph, dtype, *flags)
    te = H.tensors(M, N, K, a, b, c_eager, dtype, *flags)
    need, pref = gpu.matmul_mfma_workspace_bytes_for(tg, k_mode, tile)
    ws = torch.empty(max(pref, 256), dtype=torch.uint8, device="cuda")

    def fill_inputs(seed):
        gpu.init_test_data(a.data_ptr(), a.shape[0], a.shape[1], 4, repack, dtype, K ** -0.5, seed, H.stream_handle())
        gpu.init_test_data(b.data_ptr(), b.shape[0], b.shape[1], 4, not repack, dtype, K ** -0.5, seed + 1, H.stream_handle())

    def call(t):
        if with_ws:
            gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, k_mode, tile, H.stream_handle())
        else:
            gpu.matmul_mfma(t, k_mode, tile, H.stream_handle())

    fill_inputs(1)
    call(tg)                     # warm-up outside the capture: the kernels' one-time attribute set-up happens here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(tg)
    for replay in range(4):
        fill_inputs(100 + 7 * replay)
        c_graph.view(torch.uint8).fill_(0x7D)
        ws.fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        call(te)
        torch.cuda.synchronize()
        got, want = c_graph.cpu().numpy(), c_eager.cpu().numpy()
        assert np.isfinite(got).all(), (name, replay)
        if k_mode == gpu.K_SPLIT or "split k x" in gpu.matmul_mfma_describe(tg, k_mode, tile, pref if with_ws else 0):
            assert H.rel_err(got, want.astype(np.float64)) < 1e-5, (name, replay)   # atomics: order of additions varies
        else:
            np.testing.assert_array_equal(got, want, err_msg=f"{name} replay {replay}")


@pytest.mark.parametrize("k_splits", [1, 3])
def test_xgemm_entry_replays_correctly_from_a_graph(gpu, k_splits):
    """The fp32 entry point with the reference's Exo argument list (xgemm_Sm90.py:43-48): two conversion kernels, for
    K splits a fill kernel, and one batched GEMM launch, captured once and replayed on changing inputs."""
    L, M, N, cluster_k = 3, 200, 264, 256
    K = k_splits * cluster_k
    a = torch.empty((L, M, K), dtype=torch.float32, device="cuda")
    b = torch.empty((L, N, K), dtype=torch.float32, device="cuda")
    c_graph = torch.empty((L, N, M), dtype=torch.float32, device="cuda")
    c_eager = torch.empty_like(c_graph)
    need = gpu.xgemm_workspace_bytes(L, M, N, K, gpu.F32_BF16X3)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")

    def call(c):
        # (the context names the stream: torch captures on a stream of its own, current only inside the capture)
        ctxt = gpu.XgemmContext(ws.data_ptr(), need, H.stream_handle(), gpu.F32_BF16X3, gpu.TILE_128x128)
        gpu.xgemm_Sm90_wgmma(ctxt, L, M, N, k_splits, cluster_k, a.data_ptr(), b.data_ptr(), c.data_ptr())

    g = torch.Generator(device="cuda").manual_seed(5)
    a.normal_(generator=g)
    b.normal_(generator=g)
    call(c_graph)                # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(c_graph)
    for replay in range(4):
        a.normal_(generator=g)
        b.normal_(generator=g)
        c_graph.view(torch.uint8).fill_(0x7D)
        ws.fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        call(c_eager)
        torch.cuda.synchronize()
        got, want = c_graph.cpu().numpy(), c_eager.cpu().numpy()
        assert np.isfinite(got).all(), replay
        if k_splits > 1:
            assert H.rel_err(got, want.astype(np.float64)) < 1e-5, replay   # atomics: the order of additions varies
        else:
            np.testing.assert_array_equal(got, want, err_msg=f"replay {replay}")


_PREPARED_CAPTURE = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
import helpers as H
import spork_amd as S

torch.cuda.set_device(0)
failures = 0
S.matmul_mfma_sum_in_launch(True)   # (not the default: the captured launches then carry the library's arrival counters)
# name: (M, N, K, k_mode, tile, workspace bytes; -1: the library's own scratch array)
cases = {"output_stationary": (512, 768, 1024, S.K_OUTPUT_STATIONARY, S.TILE_256x256, 0),
         "split_k_workspace_sum": (256, 384, 4096, S.K_SPLIT_REDUCE, S.TILE_128x128, 1 << 24),
         "ragged_edge_build": (300, 504, 1000, S.K_AUTO, S.TILE_AUTO, 0),
         "stream_k": (256, 768, 21888, S.K_STREAM, S.TILE_256x256, 80 << 20),
         "static_scratch": (256, 384, 4096, S.K_SPLIT_REDUCE, S.TILE_64x128, -1)}
for name, (M, N, K, k_mode, tile, ws_bytes) in cases.items():
    a, b = H.dev_u16(M, K), H.dev_u16(N, K)
    c_graph, c_eager = H.poisoned_c(M, N), H.poisoned_c(M, N)
    tg, te = H.tensors(M, N, K, a, b, c_graph, 1), H.tensors(M, N, K, a, b, c_eager, 1)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda")

    def call(t):
        if ws_bytes < 0:
            S.matmul_mfma_static(t, k_mode, tile, H.stream_handle())
        elif ws_bytes:
            S.matmul_mfma_ws(t, ws.data_ptr(), ws_bytes, k_mode, tile, H.stream_handle())
        else:
            S.matmul_mfma(t, k_mode, tile, H.stream_handle())

    # no eager call first: only the prepare entry (and, for the static entry, the set-up call that looks up its array)
    S.matmul_mfma_prepare(tg, k_mode, tile, S.STATIC_SCRATCH_BYTES if ws_bytes < 0 else ws_bytes)
    if ws_bytes < 0:
        S.lib().mi_rt_set_device(0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(tg)
    for replay in range(3):
        for t_, seed in ((a, 10 + replay), (b, 20 + replay)):
            S.init_test_data(t_.data_ptr(), t_.shape[0], t_.shape[1], 4, t_ is b, 1, K ** -0.5, seed, H.stream_handle())
        c_graph.view(torch.uint8).fill_(0x7D)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        call(te)
        torch.cuda.synchronize()
        same = np.array_equal(c_graph.cpu().numpy().view(np.uint32), c_eager.cpu().numpy().view(np.uint32))
        print(f"{name} replay {replay}: {'same bits' if same else 'DIFFERENT'}", flush=True)
        failures += not same
# the three calls with a workspace summed their parts inside the launch, captured (once) and eager (three times)
print(f"in-launch sums: {S.matmul_mfma_sum_in_launch()[1]}", flush=True)
failures += S.matmul_mfma_sum_in_launch()[1] != 3 * 4
sys.exit(1 if failures else 0)
"""


def test_capture_preceded_only_by_prepare(gpu):
    """A first call made inside a capture works when mi_matmul_mfma_prepare has run: in a process of its own, so that no
    earlier test has launched (and thereby set up) the kernels."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", _PREPARED_CAPTURE, root], capture_output=True, text=True, timeout=110)
    print(out.stdout[-3000:], out.stderr[-3000:], flush=True)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    assert out.stdout.count("same bits") == 15
