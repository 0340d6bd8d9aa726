"""The sum of K partitions (MI_K_SPLIT_REDUCE) and of stream-K parts (MI_K_STREAM) inside the GEMM launch: the workgroup
that stores a tile's last part adds the tile's parts, in their fixed order, into C (the role of the reduce-adding epilogue
of gemm/gemm_sm90.cu:944-963, with the work generators of :1004-1095).  The arrival counters behind it live in the
library, are zero before a launch and must be zero again after it.  (The library sums with a kernel launch of its own
unless mi_matmul_mfma_sum_in_launch switches this on: measured, that is the faster way on this chip.)

The checks run in a process of their own, so that every slab of counters is free at its start and the test can tell from
the library's call count which way a call summed."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

_CHILD = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
import helpers as H
import oracle as O
import spork_amd as S

torch.cuda.set_device(0)
st = H.stream_handle()
failures = 0
S.matmul_mfma_sum_in_launch(True)   # (the library's default is the sum by a launch of its own)

def report(what, ok):
    global failures
    failures += not ok
    print(f"{what}: {'ok' if ok else 'FAILED'}", flush=True)

def in_launch_calls():
    return S.matmul_mfma_sum_in_launch()[1]

# 1. One workspace, calls of different modes, tiles and tile counts one after the other, twice over: every call finds its
#    counters at zero only if the call before it put them back.  (More tiles first, then fewer, then a different mode.)
ws = torch.empty(96 << 20, dtype=torch.uint8, device="cuda")
cases = [  # (M, N, K, mode, tile)
    (1024, 1024, 2048, S.K_SPLIT_REDUCE, S.TILE_128x128),   # 64 tiles
    (256, 768, 21888, S.K_STREAM, S.TILE_256x256),           # 3 tail tiles, leftover runs across tiles
    (256, 384, 4096, S.K_SPLIT_REDUCE, S.TILE_64x128),      # 12 tiles
    (300, 500, 1000, S.K_SPLIT_REDUCE, S.TILE_128x128),     # ragged: summed by a second launch (the range-checked build
    (33, 65, 4104, S.K_SPLIT_REDUCE, S.TILE_64x128),        #   does not carry the sum), between calls that do
    (384, 384, 7360, S.K_STREAM, S.TILE_128x128),           # 9 tail tiles
    (512, 512, 32768, S.K_SPLIT_REDUCE, S.TILE_256x256),    # rotated K walks
]
before = in_launch_calls()
for rnd in range(2):
    for M, N, K, mode, tile in cases:
        a, b = H.make_inputs(M, N, K, S.BF16, 4, 4, K ** -0.5)
        c = H.poisoned_c(M, N)
        t = H.tensors(M, N, K, a, b, c, S.BF16)
        ws.fill_(0xFF)
        S.matmul_mfma_ws(t, ws.data_ptr(), ws.numel(), mode, tile, st)
        torch.cuda.synchronize()
        ref = O.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), S.BF16)
        err = H.rel_err(c.cpu().numpy(), ref)
        report(f"round {rnd} {M}x{N}x{K} mode {mode} tile {S.tile_shape(tile)['name']} rel err {err:.2e}", err < 1e-3)
whole = sum(1 for M, N, K, mode, tile in cases if M % S.tile_shape(tile)["bm"] == 0 and N % S.tile_shape(tile)["bn"] == 0)
report("every one of those calls on whole tiles summed inside its launch", in_launch_calls() - before == 2 * whole and whole == 5)

# 2. The counters of the slab really are zero again: the last arrivals of a call are counted from zero, so a call with
#    fewer K partitions than the one before it would otherwise never see its last part.  Same tiles, 8 then 2 partitions.
M, N, K = 256, 256, 8192
a, b = H.make_inputs(M, N, K, S.F16, 3, 3, 1.0)
ref = O.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), S.F16)
for room in (8, 2, 5, 2):
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, S.F16)
    S.matmul_mfma_ws(t, ws.data_ptr(), room * M * N * 4, S.K_SPLIT_REDUCE, S.TILE_128x128, st)
    torch.cuda.synchronize()
    err = H.rel_err(c.cpu().numpy(), ref)
    report(f"room for {room} partitions, rel err {err:.2e}", err < 1e-3)

# 3. More tiles than a slab holds counters (4096): the call sums with a second launch, same bits as with the switch off.
M, N, K = 64 * 65, 128 * 64, 128
a, b = H.make_inputs(M, N, K, S.F16, 3, 3, 1.0)
big_ws = torch.empty(2 * M * N * 4, dtype=torch.uint8, device="cuda")
outs = []
for in_launch in (True, False):
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, S.F16)
    S.matmul_mfma_sum_in_launch(in_launch)
    before = in_launch_calls()
    S.matmul_mfma_ws(t, big_ws.data_ptr(), big_ws.numel(), S.K_SPLIT_REDUCE, S.TILE_64x128, st)
    torch.cuda.synchronize()
    report(f"4160 tiles, switch {in_launch}: summed by a second launch", in_launch_calls() == before)
    outs.append(c.cpu().numpy())
S.matmul_mfma_sum_in_launch(True)
ref = O.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), S.F16)
report("4160 tiles against the oracle", H.rel_err(outs[0], ref) < 1e-3)
report("4160 tiles: same bits either way", np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)))
del big_ws

# 4. More workspaces than there are slabs (256): the first ones sum inside the launch, the rest with a second launch, and
#    nobody can tell from the results.
M, N, K = 64, 128, 1024
a, b = H.make_inputs(M, N, K, S.BF16, 3, 3, 1.0)
each = 2 * M * N * 4
pool = torch.empty(300 * each, dtype=torch.uint8, device="cuda")
before, first, same = in_launch_calls(), None, True
for i in range(300):
    c = H.poisoned_c(M, N)
    t = H.tensors(M, N, K, a, b, c, S.BF16)
    S.matmul_mfma_ws(t, pool.data_ptr() + i * each, each, S.K_SPLIT_REDUCE, S.TILE_64x128, st)
    torch.cuda.synchronize()
    got = c.cpu().numpy().view(np.uint32)
    first = got if first is None else first
    same = same and np.array_equal(got, first)
took = in_launch_calls() - before
print(f"300 workspaces: {took} calls summed inside the launch", flush=True)
report("300 workspaces: between 200 and 256 slabs were still free, the rest fell back", 200 <= took <= 256)
report("300 workspaces: the same bits from every one", same)
ref = O.gemm_f64(M, N, K, H.to_host_u16(a), H.to_host_u16(b), S.BF16)
report("300 workspaces: against the oracle", H.rel_err(first.view(np.float32), ref) < 1e-3)
# ... and a workspace that has a slab keeps it: the first workspace of the pool still sums inside the launch
before = in_launch_calls()
S.matmul_mfma_ws(H.tensors(M, N, K, a, b, H.poisoned_c(M, N), S.BF16), pool.data_ptr(), each, S.K_SPLIT_REDUCE, S.TILE_64x128, st)
torch.cuda.synchronize()
report("a workspace keeps its slab", in_launch_calls() == before + 1)
sys.exit(1 if failures else 0)
"""


def test_parts_are_summed_inside_the_launch_and_counters_return_to_zero(gpu):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", _CHILD, root], capture_output=True, text=True, timeout=110)
    print(out.stdout[-6000:], out.stderr[-3000:], flush=True)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-2000:]
    assert "FAILED" not in out.stdout and out.stdout.count(": ok") >= 14 + 1 + 4 + 4 + 4
