"""mi_matmul_mfma_static: the entry point that allocates nothing (its workspace is an array inside the library).

Checked through the C ABI against mi_matmul_mfma_ws with a workspace of the same size, which makes the same plan: the
results must be the same bits (every K mode that uses the workspace adds in a fixed order), and within the parity
tolerance of the fp64 oracle.  Two calls in a row, the second on a smaller problem, so that what the first call left in
the array is there when the second runs.
"""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

TOL = 1e-3  # normalised max error against the fp64 oracle, as in every parity test


def _pair(gpu, oracle, M, N, K, dtype, layout, k_mode, ws):
    a_cm, b_cm, c_cm = layout
    a, b = H.make_inputs(M, N, K, dtype, 3, 3, 1.0, a_cm, b_cm)
    shape = (N, M) if c_cm else (M, N)
    c_static, c_ws = H.poisoned_c(*shape), H.poisoned_c(*shape)
    t_static = H.tensors(M, N, K, a, b, c_static, dtype, a_cm, b_cm, c_cm)
    t_ws = H.tensors(M, N, K, a, b, c_ws, dtype, a_cm, b_cm, c_cm)
    print(f"static entry: {M}x{N}x{K} dtype {dtype} layout {layout} k_mode {k_mode}: "
          f"{gpu.matmul_mfma_describe(t_ws, k_mode, gpu.TILE_AUTO, ws.numel())}", flush=True)
    gpu.matmul_mfma_static(t_static, k_mode, gpu.TILE_AUTO, H.stream_handle())
    gpu.matmul_mfma_ws(t_ws, ws.data_ptr(), ws.numel(), k_mode, gpu.TILE_AUTO, H.stream_handle())
    torch.cuda.synchronize()
    got, want = c_static.cpu().numpy(), c_ws.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref = oracle.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), dtype, a_cm, b_cm)
    ref = ref.T if c_cm else ref
    assert H.rel_err(got, ref) < TOL


def test_static_entry_matches_the_workspace_entry_on_two_calls_in_a_row(gpu, oracle):
    ws = torch.empty(gpu.STATIC_SCRATCH_BYTES, dtype=torch.uint8, device="cuda")
    ws.fill_(0x7D)
    # K partitions summed from copies of C in the scratch array, A re-packed into it as well (column-major A)
    _pair(gpu, oracle, 512, 384, 8192, 1, (1, 1, 0), gpu.K_SPLIT_REDUCE, ws)
    # smaller: both operands re-packed (row-major B, K not a multiple of 8), column-major C, the planner's own choice
    _pair(gpu, oracle, 200, 136, 1004, 0, (0, 0, 1), gpu.K_AUTO, ws)
    # and the first shape again after the smaller one
    _pair(gpu, oracle, 512, 384, 8192, 1, (1, 1, 0), gpu.K_SPLIT_REDUCE, ws)


def test_static_entry_refuses_what_does_not_fit(gpu):
    # re-packing a column-major 8192 x 8192 A takes 128 MiB: more than the array
    M = N = K = 8192
    a, b = H.dev_u16(K, M), H.dev_u16(N, K)
    c = torch.empty((M, N), dtype=torch.float32, device="cuda")
    t = H.tensors(M, N, K, a, b, c, 1, 1, 1, 0)
    with pytest.raises(gpu.MiGemmError) as err:
        gpu.matmul_mfma_static(t, gpu.K_AUTO, gpu.TILE_AUTO, H.stream_handle())
    assert err.value.status == 3  # MI_ERR_WORKSPACE
