"""The planner's choice against every plan that can be forced, by the clock.

For the five benchmark configurations and six shapes of the reference driver's list (gemm/gemm_main.cpp:60-117) the
launch that K_AUTO / TILE_AUTO picks must take at most 1.10x the time of the fastest forced (tile, K mode) pair (1.18x
where that pair takes under 20 us): without
a workspace against the output-stationary and atomic split-K builds of every tile, with the preferred workspace against
those plus the workspace-sum and stream-K modes.  Times are medians of HIP-event samples taken after the clocks have
settled under the same launch; the winner is re-timed back to back with the planner's launch before the assertion, so
that drift between the first and the last candidate of a shape is not charged to either, and a miss is timed a second
time before it fails.  The file sorts after the parity tests on purpose: this is a measurement by the clock, and under
`pytest -x` a miss here must not hide a parity test.

Operands are dense (the benchmark's uniform and normal distributions) for every shape.  The planner does not see the
data, and on this power-limited chip the ranking of two plans that are close can turn with it: on the reference's
mostly-zero random style the matrix cores draw less power, the clock stays up, and a plan that keeps more CUs busy gains
on one that leaves some idle to the others' power budget (1536 x 2304 x 65536: 252 workgroups of 224x256 beat 216 of
256x256 by 10 % on sparse data and tie with them on dense data).  The planner's constants were measured on dense data.
"""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

SLACK = 1.10

SHAPES = [
    # (name, M, N, K, dtype, data code, param)
    ("c1", 512, 512, 512, 0, 3, 1.0),
    ("c2", 4096, 4096, 4096, 0, 3, 1.0),
    ("c3", 8192, 8192, 8192, 1, 4, 8192 ** -0.5),
    ("c4", 16384, 128, 8192, 0, 3, 1.0),
    ("c5", 2048, 2048, 65536, 0, 3, 0.5),
    ("7680x1536x4096", 7680, 1536, 4096, 0, 3, 1.0),
    ("15360x1536x8192", 15360, 1536, 8192, 1, 4, 8192 ** -0.5),
    ("1536x2304x65536", 1536, 2304, 65536, 0, 3, 0.5),
    ("7680x3072x16384", 7680, 3072, 16384, 1, 4, 16384 ** -0.5),
    ("768x3072x3072", 768, 3072, 3072, 0, 3, 1.0),
    ("4096x4352x8192", 4096, 4352, 8192, 1, 4, 8192 ** -0.5),   # 272 tiles of 256x256: a round and a tail
]


def _median_us(launch, settle_ms=12.0, samples=9):
    """Median of `samples` HIP-event times per launch, after at least `settle_ms` of the same launch.  A sample spans as
    many launches as fill about 150 us, so that a problem of a few microseconds is not timed by the jitter of a single
    dispatch."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    elapsed, n = 0.0, 0
    while elapsed < settle_ms and n < 4000:
        for _ in range(4):
            launch()
        n += 4
        stop.record()
        stop.synchronize()
        elapsed = start.elapsed_time(stop)
    reps = max(1, min(64, int(0.150 / max(elapsed / n, 1e-4))))
    events = [torch.cuda.Event(enable_timing=True) for _ in range(samples + 1)]
    events[0].record()
    for i in range(samples):
        for _ in range(reps):
            launch()
        events[i + 1].record()
    torch.cuda.synchronize()
    return float(np.median([events[i].elapsed_time(events[i + 1]) for i in range(samples)])) * 1e3 / reps


@pytest.mark.parametrize("shape", SHAPES, ids=[s[0] for s in SHAPES])
def test_auto_is_within_a_tenth_of_the_best_forced_plan(gpu, shape):
    name, M, N, K, dtype, code, param = shape
    a = H.gen_on_device(M, K, code, False, dtype, param, 20010106)
    b = H.gen_on_device(N, K, code, True, dtype, param, 19980724)
    c = torch.empty((M, N), dtype=torch.float32, device="cuda")
    t = H.tensors(M, N, K, a, b, c, dtype)
    st = H.stream_handle()
    _, pref = gpu.matmul_mfma_workspace_bytes_for(t)
    # the largest workspace any forced plan below prefers, so that one buffer serves them all
    modes_ws = (gpu.K_SPLIT_REDUCE, gpu.K_STREAM)
    ws_bytes = max([pref, 1] + [gpu.matmul_mfma_workspace_bytes_for(t, m, tile["code"])[1] for m in modes_ws
                                for tile in gpu.tiles() if gpu.matmul_mfma_supports(t, m, tile["code"])])
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")

    def forced(mode, tile):
        if mode in modes_ws:
            size = gpu.matmul_mfma_workspace_bytes_for(t, mode, tile)[1]
            return lambda: gpu.matmul_mfma_ws(t, ws.data_ptr(), size, mode, tile, st)
        return lambda: gpu.matmul_mfma(t, mode, tile, st)

    def auto_plain():
        gpu.matmul_mfma(t, gpu.K_AUTO, gpu.TILE_AUTO, st)

    def auto_ws():
        gpu.matmul_mfma_ws(t, ws.data_ptr(), pref, gpu.K_AUTO, gpu.TILE_AUTO, st)

    for label, auto, modes in (("no workspace", auto_plain, (gpu.K_OUTPUT_STATIONARY, gpu.K_SPLIT)),
                               ("workspace", auto_ws, (gpu.K_OUTPUT_STATIONARY, gpu.K_SPLIT) + modes_ws)):
        timed = {}
        for tile in gpu.tiles():
            for mode in modes:
                if not gpu.matmul_mfma_supports(t, mode, tile["code"]):
                    continue
                try:
                    timed[(tile["code"], mode)] = _median_us(forced(mode, tile["code"]))
                except gpu.MiGemmError:
                    pass  # (a mode that the shape admits in general but not with this tile)
        assert timed, "no plan could be forced"
        best = min(timed, key=timed.get)
        described = gpu.matmul_mfma_describe(t, gpu.K_AUTO, gpu.TILE_AUTO, pref if auto is auto_ws else 0)
        # (under 20 us the dispatch is a third of the time and its spread between two measurements several per cent)
        ratio, auto_us, best_us = 0.0, 0.0, 0.0
        for attempt in range(2):
            # back to back: the winner, the planner's launch, the winner again
            first = _median_us(forced(best[1], best[0]))
            auto_us = _median_us(auto)
            second = _median_us(forced(best[1], best[0]))
            best_us = min(first, second, timed[best]) if attempt == 0 else min(first, second)
            slack = SLACK if best_us >= 20.0 else SLACK + 0.08
            ratio = auto_us / best_us
            print(f"{name} ({label}): auto {auto_us:.1f} us [{described}]; best forced {gpu.tile_shape(best[0])['name']} "
                  f"mode {best[1]} {best_us:.1f} us; ratio {ratio:.3f}" + ("" if ratio <= slack else "  <- over, timed again"))
            if ratio <= slack:
                break
            # One noisy sample (a clock dip, a neighbour on the box) must not fail the suite: the three are timed once
            # more, this time against the winner's times of this pass alone.
        print("  every forced plan, us: " + ", ".join(f"{gpu.tile_shape(k[0])['name']}/{k[1]} {v:.1f}"
                                                         for k, v in sorted(timed.items(), key=lambda kv: kv[1])))
        assert ratio <= slack, (name, label, described, best, auto_us, best_us, sorted(timed.items(), key=lambda kv: kv[1])[:4])
