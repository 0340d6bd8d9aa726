"""CPU-side checks of the product: the C-ABI library loads and exports every symbol include/mi_gemm.h declares, the
argument validation and the support predicate / planner behave (no compute calls: there is no GPU here), the host
driver was built, and nothing in the product reaches for the oracle."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

import spork_amd as S

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _t(M, N, K, dtype=S.F16, a=256, b=512, c=1024, **kw):
    return S.GpuTensors.make(M, N, K, a, b, c, dtype, **kw)


def test_library_exports_every_declared_symbol():
    lib = S.lib()
    names = S.exported_symbols()
    assert len(names) >= 25
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    out = subprocess.run(["nm", "-D", "--defined-only", S.lib_path()], capture_output=True, text=True, check=True).stdout
    for n in names:
        assert re.search(rf"\bT {n}\b", out), n


def test_vendor_library_exports_its_header():
    from spork_amd import vendor as V

    names = V.exported_symbols()
    assert names == ["mi_vendor_accepts_algorithm", "mi_vendor_enabled", "mi_vendor_last_status", "mi_vendor_library",
                     "mi_vendor_matmul", "mi_vendor_version"]
    out = subprocess.run(["nm", "-D", "--defined-only", V.lib_path()], capture_output=True, text=True, check=True).stdout
    for n in names:
        assert re.search(rf"\bT {n}\b", out), n
    # the product library itself must not depend on a BLAS library
    needed = subprocess.run(["readelf", "-d", S.lib_path()], capture_output=True, text=True, check=True).stdout
    assert "blas" not in needed.lower()
    lib = V.lib()
    assert lib.mi_vendor_matmul(None, None, 0, None) == 2
    t = _t(0, 4, 4)
    assert lib.mi_vendor_matmul(C.byref(t), None, 0, None) == 2
    # the comparator never runs without a workspace: refused before anything touches a device
    t = _t(64, 64, 64)
    assert lib.mi_vendor_matmul(C.byref(t), None, 0, None) == 3
    assert lib.mi_vendor_matmul(C.byref(t), 4096, (32 << 20) - 1, None) == 3
    # an algorithm is kept only if the heuristic reported it usable and its workspace fits what the caller gave
    assert lib.mi_vendor_accepts_algorithm(0, 0, 32 << 20) == 0
    assert lib.mi_vendor_accepts_algorithm(0, 32 << 20, 32 << 20) == 0
    assert lib.mi_vendor_accepts_algorithm(0, (32 << 20) + 1, 32 << 20) == 3      # wants more room than there is
    assert lib.mi_vendor_accepts_algorithm(0, 128 << 20, 0) == 3
    assert lib.mi_vendor_accepts_algorithm(7, 0, 128 << 20) == 1                  # heuristic state not success
    # the comparator names the hipBLASLt it is bound to (no device needed)
    assert lib.mi_vendor_library(None, 0) == 2
    path = V.library()
    assert os.path.isfile(path) and "hipblaslt" in os.path.basename(path), path


def test_headers_are_plain_c(tmp_path):
    """The boundary is a C ABI: both public headers compile as strict C99 on their own."""
    src = tmp_path / "abi.c"
    src.write_text('#include "mi_gemm.h"\n#include "mi_gemm_vendor.h"\n'
                   "int main(void) { mi_gemm_tensors t; mi_xgemm_context x; (void)t; (void)x; return 0; }\n")
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", include, "-c", str(src), "-o",
                        str(tmp_path / "abi.o")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_struct_layout_matches_the_header():
    # uint32 x3, three pointers (8-aligned after 12 bytes -> offset 16), four uint8, padded to 8
    assert S.GpuTensors.M.offset == 0 and S.GpuTensors.K.offset == 8
    assert S.GpuTensors.a.offset == 16 and S.GpuTensors.c.offset == 32
    assert S.GpuTensors.a_col_major.offset == 40 and S.GpuTensors.ab_dtype.offset == 43
    assert C.sizeof(S.GpuTensors) == 48


def test_status_strings():
    assert S.status_string(0) == "ok"
    assert "unsupported" in S.status_string(1)
    assert S.status_string(12345) == "unknown status"


def test_argument_validation_without_a_gpu():
    lib = S.lib()
    assert lib.mi_matmul_mfma(None, 0, 0, None) == 2
    assert lib.mi_matmul_baseline(None, None) == 2
    t = _t(256, 256, 256, a=0)
    assert lib.mi_matmul_mfma(C.byref(t), S.K_AUTO, S.TILE_AUTO, None) == 2      # null A
    t = _t(0, 256, 256)
    assert lib.mi_matmul_mfma(C.byref(t), S.K_AUTO, S.TILE_AUTO, None) == 2      # zero size
    t = _t(256, 256, 256, dtype=7)
    assert lib.mi_matmul_mfma(C.byref(t), S.K_AUTO, S.TILE_AUTO, None) == 2      # unknown dtype
    t = _t(256, 256, 256)
    assert lib.mi_matmul_mfma(C.byref(t), 9, S.TILE_AUTO, None) == 2             # unknown k mode
    assert lib.mi_matmul_mfma(C.byref(t), S.K_AUTO, 99, None) == 2               # unknown tile
    t = _t(100, 100, 100)
    assert lib.mi_matmul_mfma(C.byref(t), S.K_AUTO, S.TILE_AUTO, None) == 1      # no tile divides it
    assert lib.mi_matmul_mfma_direct(C.byref(t), None) == 1
    assert lib.mi_init_test_data(None, 4, 4, 0, 0, 0, 1.0, 0, None) == 2
    assert lib.mi_compare_tensors(None, None, 4, 4, None, None) == 2


def test_supports_predicate():
    # canonical layout of the testbed: A row-major, B stored N x K (gemm/gemm_test.cu:305,365)
    assert S.matmul_mfma_supports(_t(8192, 8192, 8192, S.BF16))
    assert S.matmul_mfma_supports(_t(128, 128, 32))
    # ragged M and N and a K that is only a multiple of 8 go through the bounds-checked build
    assert S.matmul_mfma_supports(_t(160, 480, 816))
    assert S.matmul_mfma_supports(_t(1, 1, 8))
    assert S.matmul_mfma_supports(_t(64, 64, 64))
    assert S.matmul_mfma_supports(_t(64, 256, 256, c_col_major=1))
    assert not S.matmul_mfma_supports(_t(256, 256, 100))              # rows are not whole 16-byte chunks
    assert not S.matmul_mfma_supports(_t(256, 256, 256, a_col_major=1))
    assert not S.matmul_mfma_supports(_t(256, 256, 256, b_col_major=0))
    assert not S.matmul_mfma_supports(_t(256, 256, 256, a=260))       # A not 16-byte aligned
    # the range-checked build counts rows in signed 32-bit integers: 2^31 rows and more are refused, on either side
    assert S.matmul_mfma_supports(_t((1 << 31) - 8, 8, 8))
    assert not S.matmul_mfma_supports(_t(1 << 31, 8, 8))
    assert not S.matmul_mfma_supports(_t(8, 1 << 31, 8, c_col_major=1))
    assert not S.matmul_mfma_supports(_t(8, 1 << 21, 8))              # N beyond a descriptor's 32-bit offsets
    # explicit tiles
    assert S.matmul_mfma_supports(_t(256, 256, 64), S.K_OUTPUT_STATIONARY, S.TILE_256x256)
    assert S.matmul_mfma_supports(_t(128, 256, 64), S.K_OUTPUT_STATIONARY, S.TILE_256x256)
    # a single K tile cannot be split: MI_K_SPLIT then degenerates to one partition (no atomics)
    assert S.matmul_mfma_plan(_t(256, 256, 64), S.K_SPLIT, S.TILE_256x256)["k_splits"] == 1
    assert S.matmul_mfma_plan(_t(256, 256, 128), S.K_SPLIT, S.TILE_256x256)["k_splits"] == 2


def test_tile_family_is_enumerated_from_the_library():
    """One table in the library defines the tile family; the binding's TILE_* names come from the header's enumerators
    and shapes, names and the count from mi_tile_count / mi_tile_name / mi_tile_shape: they must agree."""
    tiles = S.tiles()
    assert len(tiles) == S.tile_count() - 1 == len(S.TILE_CODES) - 1
    for t in tiles:
        assert S.TILE_CODES[f"TILE_{t['name']}"] == t["code"]
        assert t["name"] == f"{t['bm']}x{t['bn']}" and t["workgroups_per_cu"] in (1, 2)
        # every tile is accepted when forced on a problem of whole tiles, and named by the plan
        plan = S.matmul_mfma_plan(_t(2 * t["bm"], 3 * t["bn"], 256), S.K_OUTPUT_STATIONARY, t["code"])
        assert plan["tile"] == t["name"] and plan["tile_code"] == t["code"]
    assert S.lib().mi_tile_name(0) == b"auto" and S.lib().mi_tile_name(S.tile_count()) == b"unknown"
    assert S.lib().mi_tile_shape(0, None, None, None, None) == 2
    assert S.lib().mi_tile_shape(S.tile_count(), None, None, None, None) == 2
    assert [t["name"] for t in tiles if t["has_32_deep_twin"]] == ["256x256", "256x128", "128x128", "64x128", "192x256"]
    assert [t["name"] for t in tiles if t["workgroups_per_cu"] == 2] == ["192x128"]


def test_prepare_entry_validates_like_the_call_it_prepares():
    lib = S.lib()
    assert lib.mi_matmul_mfma_prepare(None, S.K_AUTO, S.TILE_AUTO, 0) == 2
    assert lib.mi_matmul_mfma_prepare(C.byref(_t(256, 256, 256)), 9, S.TILE_AUTO, 0) == 2
    assert lib.mi_matmul_mfma_prepare(C.byref(_t(256, 256, 100)), S.K_AUTO, S.TILE_AUTO, 0) == 1       # needs re-packing
    assert lib.mi_matmul_mfma_prepare(C.byref(_t(256, 256, 100)), S.K_AUTO, S.TILE_AUTO, 4096) == 3    # too little room


def test_workspace_size_query():
    lib = S.lib()
    assert S.matmul_mfma_workspace_bytes(_t(8192, 8192, 8192, S.BF16)) == 0          # read in place
    assert S.matmul_mfma_workspace_bytes(_t(160, 480, 816, c_col_major=1)) == 0      # C layout never needs a copy
    # row-major B (K x N) is re-packed to N x K; A stays in place
    assert S.matmul_mfma_workspace_bytes(_t(256, 512, 128, b_col_major=0)) == 512 * 128 * 2
    # column-major A (K x M) likewise
    assert S.matmul_mfma_workspace_bytes(_t(256, 512, 128, a_col_major=1)) == 256 * 128 * 2
    # K = 100 is padded to 104 for both operands; each region is rounded up to 256 bytes
    need = S.matmul_mfma_workspace_bytes(_t(300, 200, 100))
    up = lambda x: (x + 255) // 256 * 256
    assert need == up(300 * 104 * 2) + up(200 * 104 * 2)
    # a misaligned pointer is copied too
    assert S.matmul_mfma_workspace_bytes(_t(64, 64, 64, a=260)) == 64 * 64 * 2
    n = C.c_size_t()
    assert lib.mi_matmul_mfma_workspace_bytes(None, C.byref(n)) == 2
    t = _t(64, 64, 64)
    assert lib.mi_matmul_mfma_workspace_bytes(C.byref(t), None) == 2
    # the workspace entry point validates before touching a device
    t = _t(300, 200, 100)
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_AUTO, S.TILE_AUTO, None, 0, None) == 3         # workspace missing
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_AUTO, S.TILE_AUTO, 4096, need - 1, None) == 3  # too small
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_AUTO, S.TILE_AUTO, 4100, need, None) == 3      # workspace not 256-byte aligned
    assert lib.mi_matmul_mfma_ws(None, 0, 0, None, 0, None) == 2


def test_workspace_sum_of_k_partitions_sizes_and_validation():
    """MI_K_SPLIT_REDUCE: the partitions' private copies of C live in the caller's workspace."""
    lib = S.lib()
    up = lambda x: (x + 255) // 256 * 256
    # deep K, few tiles: with room the planner prefers the workspace sum and asks for k_splits copies of C
    t = _t(1536, 2304, 65536)
    forced = S.matmul_mfma_plan(t, S.K_SPLIT_REDUCE)
    assert forced["k_mode"] == "split k (workspace sum)" and forced["k_splits"] > 1
    req, pref = S.matmul_mfma_workspace_bytes_for(t, S.K_SPLIT_REDUCE)
    assert pref == forced["k_splits"] * 1536 * 2304 * 4 and req == 2 * 1536 * 2304 * 4   # two partitions at least
    req, pref = S.matmul_mfma_workspace_bytes_for(t, S.K_AUTO)
    auto = S.matmul_mfma_describe(t, S.K_AUTO, S.TILE_AUTO, pref)
    # (the planner's own choice with room is one of the two modes that use it: copies of C, or stream-K parts)
    assert req == 0 and pref > 0 and ("stream k" in auto or pref % (1536 * 2304 * 4) == 0), auto
    # without a workspace the same call falls back to atomics; the plan query (no workspace) says so
    assert S.matmul_mfma_plan(t)["k_mode"] == "split k"
    # a problem that fills the chip unsplit prefers no workspace at all
    assert S.matmul_mfma_workspace_bytes_for(_t(8192, 8192, 8192, S.BF16)) == (0, 0)
    # re-packed operands come first, each copy region 256-byte aligned
    t = _t(300, 200, 4000, b_col_major=0)
    req, pref = S.matmul_mfma_workspace_bytes_for(t, S.K_SPLIT_REDUCE)
    splits = (pref - up(200 * 4000 * 2)) // (300 * 200 * 4)
    assert splits > 1 and pref == up(200 * 4000 * 2) + splits * 300 * 200 * 4
    assert req == up(200 * 4000 * 2) + 2 * 300 * 200 * 4
    # forced mode without enough room is a workspace error, before any launch
    t = _t(1536, 2304, 65536)
    need = S.matmul_mfma_workspace_bytes_for(t, S.K_SPLIT_REDUCE)[0]
    assert lib.mi_matmul_mfma(C.byref(t), S.K_SPLIT_REDUCE, S.TILE_AUTO, None) == 3
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_SPLIT_REDUCE, S.TILE_AUTO, None, 0, None) == 3
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_SPLIT_REDUCE, S.TILE_AUTO, 4096, 1 << 20, None) == 3
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_SPLIT_REDUCE, S.TILE_AUTO, 4096, need - 1, None) == 3
    assert lib.mi_matmul_mfma_ws(C.byref(t), S.K_SPLIT_REDUCE, S.TILE_AUTO, 4100, need, None) == 3  # misaligned
    # stream-K: whole tiles, a tile count that does not fill whole rounds of CUs.  44 tiles on 256 CUs (what the library
    # assumes when no device is visible, and what an MI355X has): 5 main partitions per tile, 36 leftover workgroups,
    # 44 * 5 + 36 + 44 - 1 parts
    t = _t(1024, 2816, 49152)
    sk = S.matmul_mfma_plan(t, S.K_STREAM, S.TILE_256x256)
    assert sk["k_mode"] == "stream k" and sk["k_splits"] == 1
    assert S.matmul_mfma_workspace_bytes_for(t, S.K_STREAM, S.TILE_256x256) == (299 * 256 * 256 * 4,) * 2
    assert lib.mi_matmul_mfma(C.byref(t), S.K_STREAM, S.TILE_AUTO, None) == 3                 # needs the workspace
    assert not S.matmul_mfma_supports(_t(8192, 8192, 8192), S.K_STREAM)                       # whole rounds with every tile
    assert S.matmul_mfma_supports(_t(8192 + 256, 8192, 8192), S.K_STREAM, S.TILE_256x256)     # four rounds and 32 tiles
    assert not S.matmul_mfma_supports(_t(1000, 2816, 49152), S.K_STREAM)                      # ragged M
    assert not S.matmul_mfma_supports(_t(1024, 2816, 49152 + 8), S.K_STREAM)                  # K not a multiple of 64
    assert S.matmul_mfma_plan(t)["k_mode"] != "stream k"                                      # not without a workspace
    # argument checks of the query
    a, b = C.c_size_t(), C.c_size_t()
    assert lib.mi_matmul_mfma_workspace_bytes_for(None, S.K_AUTO, S.TILE_AUTO, C.byref(a), C.byref(b)) == 2
    assert lib.mi_matmul_mfma_workspace_bytes_for(C.byref(t), S.K_AUTO, S.TILE_AUTO, None, C.byref(b)) == 2
    assert lib.mi_matmul_mfma_workspace_bytes_for(C.byref(t), S.K_AUTO, S.TILE_AUTO, C.byref(a), None) == 2
    assert lib.mi_matmul_mfma_workspace_bytes_for(C.byref(t), 5, S.TILE_AUTO, C.byref(a), C.byref(b)) == 2
    # a single K tile cannot be split: the forced mode degenerates to one output-stationary partition
    assert S.matmul_mfma_plan(_t(256, 256, 64), S.K_SPLIT_REDUCE)["k_splits"] == 1
    assert S.matmul_mfma_workspace_bytes_for(_t(256, 256, 64), S.K_SPLIT_REDUCE) == (0, 0)


def test_describe_and_peeling_decisions():
    """The text form of the plan: one launch, K partitions, or a ragged problem peeled into whole tiles plus strips."""
    lib = S.lib()
    assert S.matmul_mfma_describe(_t(8192, 8192, 8192, S.BF16)) == "8192x8192x8192 256x256 output stationary"
    assert S.matmul_mfma_describe(_t(1024, 2816, 49152)) == "1024x2816x49152 256x256 split k x5"
    assert S.matmul_mfma_describe(_t(1024, 2816, 49152), workspace_bytes=1 << 30) == \
        "1024x2816x49152 256x256 split k (workspace sum) x5"
    # the estimate the planner ranks by: the headline is priced within 15 % of what it measures (0.71-0.76 ms), and
    # a forced plan is never priced below the planner's own choice
    assert 650.0 < S.matmul_mfma_estimate_us(_t(8192, 8192, 8192, S.BF16)) < 820.0
    best = S.matmul_mfma_estimate_us(_t(1024, 2816, 49152), workspace_bytes=1 << 30)
    for tile in range(1, 14):
        assert S.matmul_mfma_estimate_us(_t(1024, 2816, 49152), S.K_SPLIT_REDUCE, tile, 1 << 30) >= best
    assert lib.mi_matmul_mfma_estimate_us(C.byref(_t(64, 64, 64)), 0, 0, 0, None) == 2
    # eight rows over a multiple of the tile: the whole tiles keep the plain 256x256 kernel
    text = S.matmul_mfma_describe(_t(8200, 8192, 8192, S.BF16))
    assert text.startswith("peeled: ") and " output stationary + bottom " in text and "right" not in text, text
    # 272 tiles of 256x256 on 256 CUs: one whole round, then the last tile column as a launch of its own
    text = S.matmul_mfma_describe(_t(4096, 4352, 8192, S.BF16))
    assert text.startswith("peeled: 4096x4096x8192 256x256 output stationary + right 4096x256x8192 "), text
    text = S.matmul_mfma_describe(_t(40016, 32768, 6400, S.BF16))   # gemm/gemm_main.cpp:109
    assert text.startswith("peeled: 39") and " output stationary + bottom " in text and "right" not in text, text
    # the tile that puts two workgroups on a CU is the planner's for short K only (measured behind from K = 1536 on),
    # whole problems and the whole-tile part of a peeled one alike; a caller can still force it
    assert " 192x128 " in S.matmul_mfma_describe(_t(7072, 7352, 1024, S.BF16))
    for shape in ((3000, 11008, 4096), (4592, 2160, 8192), (7072, 7352, 2048)):
        assert "192x128" not in S.matmul_mfma_describe(_t(*shape, S.BF16)), shape
    assert " 192x128 " in S.matmul_mfma_describe(_t(3000, 11008, 4096, S.BF16), S.K_OUTPUT_STATIONARY, S.TILE_192x128)
    # a 64-row tile on rows of K that straddle cache lines is dear (one launch of it measured 28 us here, K
    # partitions of it or of the 128x128 tile 22 to 25 us)
    assert " split k x" in S.matmul_mfma_describe(_t(512, 1312, 3432, S.BF16))
    # a problem of a few microseconds is not worth a second launch that sums partitions
    assert S.matmul_mfma_describe(_t(160, 480, 816), workspace_bytes=1 << 30) == "160x480x816 64x128 output stationary"
    # not peeled: a short ragged K on a problem whose tiles fill the rounds anyway, N not a multiple of 4 (the plain
    # kernel stores 16 bytes), a forced tile (the caller asked for one launch of it), small problems (the extra
    # launches cost more than they save)
    assert "peeled" not in S.matmul_mfma_describe(_t(32768, 40016, 816, S.BF16))
    assert "peeled" not in S.matmul_mfma_describe(_t(8192, 8198, 8192))
    assert "peeled" not in S.matmul_mfma_describe(_t(8200, 8192, 8192), S.K_AUTO, S.TILE_256x256)
    assert "peeled" not in S.matmul_mfma_describe(_t(300, 500, 1024))
    # re-packed operands are named; too small a workspace is an error
    assert S.matmul_mfma_describe(_t(300, 200, 100, b_col_major=0, a_col_major=1), workspace_bytes=1 << 20).startswith("re-pack A and B, then ")
    buf = C.create_string_buffer(64)
    t = _t(300, 200, 100, b_col_major=0)
    assert lib.mi_matmul_mfma_describe(C.byref(t), S.K_AUTO, S.TILE_AUTO, 0, buf, 64) == 1
    assert lib.mi_matmul_mfma_describe(C.byref(t), S.K_AUTO, S.TILE_AUTO, 256, buf, 64) == 3
    t = _t(8200, 8192, 8192)
    assert lib.mi_matmul_mfma_describe(C.byref(t), S.K_AUTO, S.TILE_AUTO, 0, None, 64) == 2
    assert lib.mi_matmul_mfma_describe(C.byref(t), S.K_AUTO, S.TILE_AUTO, 0, buf, 0) == 2
    assert lib.mi_matmul_mfma_describe(None, S.K_AUTO, S.TILE_AUTO, 0, buf, 64) == 2
    small = C.create_string_buffer(16)   # truncated, still terminated
    assert lib.mi_matmul_mfma_describe(C.byref(t), S.K_AUTO, S.TILE_AUTO, 0, small, 16) == 0
    assert len(small.value) == 15 and small.value.startswith(b"peeled: ")


def test_planner_queries_from_many_threads_agree():
    """The planner keeps per-thread memos; concurrent callers must get the answers a single thread gets."""
    import threading

    shapes = [(8192, 8192, 8192), (1024, 2816, 49152), (8200, 8192, 8192), (5000, 1024, 8192), (160, 480, 816),
              (2048, 2048, 65536), (300, 500, 1000), (40016, 32768, 6400)]
    expected = {sh: (S.matmul_mfma_describe(_t(*sh)), S.matmul_mfma_describe(_t(*sh), workspace_bytes=1 << 30),
                     S.matmul_mfma_workspace_bytes_for(_t(*sh))) for sh in shapes}
    failures = []

    def worker(seed):
        order = shapes[seed % len(shapes):] + shapes[:seed % len(shapes)]
        for _ in range(25):
            for sh in order:
                got = (S.matmul_mfma_describe(_t(*sh)), S.matmul_mfma_describe(_t(*sh), workspace_bytes=1 << 30),
                       S.matmul_mfma_workspace_bytes_for(_t(*sh)))
                if got != expected[sh]:
                    failures.append((sh, got))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures[:3]


def test_batched_entry_validates_its_arguments():
    lib = S.lib()
    t = _t(256, 256, 256)
    assert lib.mi_matmul_mfma_batched(None, 2, 0, 0, 0, S.K_AUTO, S.TILE_AUTO, None) == 2
    assert lib.mi_matmul_mfma_batched(C.byref(t), 0, 0, 0, 0, S.K_AUTO, S.TILE_AUTO, None) == 2          # no problems
    assert lib.mi_matmul_mfma_batched(C.byref(t), 2, 0, 0, 256 * 256 - 1, S.K_AUTO, S.TILE_AUTO, None) == 2  # C overlap
    assert lib.mi_matmul_mfma_batched(C.byref(t), 2, 256 * 256 + 4, 0, 0, S.K_AUTO, S.TILE_AUTO, None) == 1  # A stride % 8
    t = _t(256, 256, 256, b_col_major=0)
    assert lib.mi_matmul_mfma_batched(C.byref(t), 2, 0, 0, 0, S.K_AUTO, S.TILE_AUTO, None) == 1          # needs re-packing


def test_f32_entry_sizes_and_validation():
    lib = S.lib()
    up = lambda x: (x + 255) // 256 * 256
    t = _t(300, 200, 100, dtype=S.F32)
    # K = 100 pads to 104 per term; three terms per row for the split, one for plain rounding
    assert S.matmul_f32_workspace_bytes(t, S.F32_BF16X3) == up(300 * 312 * 2) + up(200 * 312 * 2)
    assert S.matmul_f32_workspace_bytes(t, S.F32_BF16X1) == up(300 * 104 * 2) + up(200 * 104 * 2)
    n = C.c_size_t()
    assert lib.mi_matmul_f32_workspace_bytes(C.byref(t), 7, C.byref(n)) == 2            # unknown precision
    t16 = _t(300, 200, 100)
    assert lib.mi_matmul_f32_workspace_bytes(C.byref(t16), S.F32_BF16X3, C.byref(n)) == 2   # wants MI_F32
    assert lib.mi_matmul_mfma(C.byref(t), S.K_AUTO, S.TILE_AUTO, None) == 2              # and the 16-bit entry refuses it
    need = S.matmul_f32_workspace_bytes(t, S.F32_BF16X3)
    assert lib.mi_matmul_f32_ws(C.byref(t), S.F32_BF16X3, S.K_AUTO, S.TILE_AUTO, None, 0, None) == 3
    assert lib.mi_matmul_f32_ws(C.byref(t), S.F32_BF16X3, S.K_AUTO, S.TILE_AUTO, 4096, need - 1, None) == 3
    assert lib.mi_matmul_f32_ws(C.byref(t), S.F32_BF16X3, 9, S.TILE_AUTO, 4096, need, None) == 2


def test_xgemm_entries_sizes_and_validation():
    """The entry points with the argument lists of the reference's Exo-generated C (xgemm_Sm80.py:18-21,
    xgemm_Sm90.py:43-54): what they refuse before any device call."""
    lib = S.lib()
    up = lambda x: (x + 255) // 256 * 256
    # the shape of the reference's own sync check (xgemm_Sm90.py:203): L = 2, M = 500, N = 800, K = 2 * 240
    assert S.xgemm_workspace_bytes(2, 500, 800, 480) == up(2 * 500 * 1440 * 2) + up(2 * 800 * 1440 * 2)
    assert S.xgemm_workspace_bytes(1, 500, 800, 480, S.F32_BF16X1) == up(500 * 480 * 2) + up(800 * 480 * 2)
    n = C.c_size_t()
    for bad in ((0, 8, 8, 8), (1, 0, 8, 8), (1, 8, -1, 8), (1, 8, 8, 0)):
        assert lib.mi_xgemm_workspace_bytes(*bad, S.F32_BF16X3, C.byref(n)) == 2, bad
    assert lib.mi_xgemm_workspace_bytes(1, 8, 8, 8, S.F32_BF16X3, None) == 2
    assert lib.mi_xgemm_workspace_bytes(1, 8, 8, 8, 5, C.byref(n)) == 2
    assert C.sizeof(S.XgemmContext) == 32 and S.XgemmContext.precision.offset == 24 and S.XgemmContext.tile.offset == 28
    need = S.xgemm_workspace_bytes(1, 192, 256, 64)
    ctxt = S.XgemmContext(4096, need, None, S.F32_BF16X3, S.TILE_AUTO)
    p = 4096  # placeholder addresses: every call below is refused before anything is launched
    # a null context is the reference's call form (gemm/gemm_test.cu:326,335): the library's resident scratch stands in,
    # so what does not fit its 64 MiB is refused by size, and bad sizes are refused as with a context
    assert lib.mi_xgemm_Sm80(None, 8192, 8192, 8192, p, p, p) == 3
    assert lib.mi_xgemm_Sm90_wgmma(None, 1, 8192, 8192, 1, 8192, p, p, p) == 3
    assert lib.mi_xgemm_Sm90_wgmma(None, 8, 1024, 1024, 1, 1024, p, p, p) == 3         # eight problems of 12 MiB each
    assert lib.mi_xgemm_Sm80(None, 0, 256, 64, p, p, p) == 2
    assert lib.mi_xgemm_Sm80(None, 192, 256, 64, None, p, p) == 2
    assert lib.mi_xgemm_Sm80(C.byref(ctxt), 0, 256, 64, p, p, p) == 2
    assert lib.mi_xgemm_Sm80(C.byref(ctxt), 192, 256, 64, None, p, p) == 2
    assert lib.mi_xgemm_Sm90_wgmma(None, 0, 192, 256, 1, 64, p, p, p) == 2
    assert lib.mi_xgemm_Sm90_wgmma(C.byref(ctxt), 0, 192, 256, 1, 64, p, p, p) == 2
    assert lib.mi_xgemm_Sm90_wgmma(C.byref(ctxt), 1, 192, 256, 0, 64, p, p, p) == 2
    assert lib.mi_xgemm_Sm90_wgmma(C.byref(ctxt), 1, 192, 256, 1, 0, p, p, p) == 2
    small = S.XgemmContext(4096, need - 1, None, S.F32_BF16X3, S.TILE_AUTO)
    assert lib.mi_xgemm_Sm80(C.byref(small), 192, 256, 64, p, p, p) == 3
    assert lib.mi_xgemm_Sm90_wgmma(C.byref(small), 1, 192, 256, 1, 64, p, p, p) == 3
    assert lib.mi_xgemm_Sm90_wgmma(C.byref(ctxt), 2, 192, 256, 1, 64, p, p, p) == 3   # two problems need twice the room
    unaligned = S.XgemmContext(4096 + 64, need, None, S.F32_BF16X3, S.TILE_AUTO)
    assert lib.mi_xgemm_Sm80(C.byref(unaligned), 192, 256, 64, p, p, p) == 3
    bad_tile = S.XgemmContext(4096, need, None, S.F32_BF16X3, 99)
    assert lib.mi_xgemm_Sm80(C.byref(bad_tile), 192, 256, 64, p, p, p) == 2
    assert lib.mi_widen_to_f32(None, S.BF16, p, 16, None) == 2
    assert lib.mi_widen_to_f32(p, S.F32, p, 16, None) == 2
    assert lib.mi_widen_to_f32(p, S.F16, p, 0, None) == 2


def test_ceiling_probe_validates_its_arguments():
    lib = S.lib()
    n, f = C.c_uint32(), C.c_double()
    assert lib.mi_mfma_ceiling(None, 1 << 26, S.BF16, 16, 10, 4096, 8192, C.byref(n), C.byref(f), None) == 2
    assert lib.mi_mfma_ceiling(4096, 1 << 26, S.BF16, 24, 10, 4096, 8192, C.byref(n), C.byref(f), None) == 2   # MFMA tile
    assert lib.mi_mfma_ceiling(4096, 1 << 26, S.F32, 16, 10, 4096, 8192, C.byref(n), C.byref(f), None) == 2    # 16-bit only
    assert lib.mi_mfma_ceiling(4096, 1 << 26, S.BF16, 16, 0, 4096, 8192, C.byref(n), C.byref(f), None) == 2    # no work
    assert lib.mi_mfma_ceiling(4100, 1 << 26, S.BF16, 16, 10, 4096, 8192, C.byref(n), C.byref(f), None) == 2   # alignment


def test_streaming_probes_validate_their_arguments():
    lib = S.lib()
    p = 4096
    assert lib.mi_hbm_stream_ceiling(None, p, 1 << 20, S.STREAM_READ, 1, p, None) == 2
    assert lib.mi_hbm_stream_ceiling(p + 4, p, 1 << 20, S.STREAM_READ, 1, p, None) == 2      # alignment
    assert lib.mi_hbm_stream_ceiling(p, p, 512, S.STREAM_READ, 1, p, None) == 2              # too few bytes
    assert lib.mi_hbm_stream_ceiling(p, p, 1 << 20, 3, 1, p, None) == 2                      # unknown mode
    assert lib.mi_hbm_stream_ceiling(p, p, 1 << 20, S.STREAM_READ, 0, p, None) == 2
    assert lib.mi_hbm_stream_ceiling(p, p, 1 << 20, S.STREAM_READ, 9, p, None) == 2
    assert lib.mi_hbm_stream_ceiling(p, None, 1 << 20, S.STREAM_COPY, 1, p, None) == 2       # a copy needs somewhere to go
    assert lib.mi_hbm_stream_ceiling(p, p, 1 << 20, S.STREAM_READ, 1, None, None) == 2       # and a read its sink
    assert lib.mi_hbm_stream_rows_ceiling(None, 1024, 4096, 64, None) == 2
    assert lib.mi_hbm_stream_rows_ceiling(p, 1024, 4096 + 64, 64, None) == 2                 # rows of whole 128-byte pieces
    assert lib.mi_hbm_stream_rows_ceiling(p, 1024, 4096, 60, None) == 2                      # eight rows per instruction
    assert lib.mi_hbm_stream_rows_ceiling(p, 32, 4096, 64, None) == 2                        # more rows per workgroup than rows
    assert lib.mi_hbm_stream_rows_ceiling(p, 1 << 20, 1 << 16, 1 << 15, None) == 1           # beyond one descriptor's reach


def test_static_entry_checks_arguments_and_size_before_touching_the_device():
    """mi_matmul_mfma_static refuses bad modes and operands whose re-packed copies exceed its scratch array before it
    makes any HIP call, so the refusals can be checked without a GPU."""
    lib = S.lib()
    assert S.STATIC_SCRATCH_BYTES == 64 << 20
    header = open(os.path.join(os.path.dirname(S.lib_path()), "..", "..", "include", "mi_gemm.h")).read()
    assert re.search(r"#define\s+MI_STATIC_SCRATCH_BYTES\s+\(\(size_t\)64 << 20\)", header)
    assert lib.mi_matmul_mfma_static(None, S.K_AUTO, S.TILE_AUTO, None) == 2
    assert lib.mi_matmul_mfma_static(C.byref(_t(256, 256, 256)), 9, S.TILE_AUTO, None) == 2
    # a column-major 8192 x 8192 A re-packs into 128 MiB, a 4096 x 4096 one into 32 MiB + 32 MiB for row-major B: fits
    t = _t(8192, 8192, 8192, S.BF16, a_col_major=1)
    assert lib.mi_matmul_mfma_static(C.byref(t), S.K_AUTO, S.TILE_AUTO, None) == 3
    assert S.matmul_mfma_workspace_bytes(_t(4096, 4096, 4096, S.BF16, a_col_major=1, b_col_major=0)) == 64 << 20


def test_timeline_entry_validates_its_buffer():
    lib = S.lib()
    t = _t(256, 256, 256)
    n = C.c_uint32()
    assert lib.mi_matmul_mfma_timeline(C.byref(t), S.K_AUTO, S.TILE_AUTO, None, 8, 16, C.byref(n), None) == 2
    assert lib.mi_matmul_mfma_timeline(C.byref(t), S.K_AUTO, S.TILE_AUTO, 4096, 0, 16, C.byref(n), None) == 2
    assert lib.mi_matmul_mfma_timeline(C.byref(t), S.K_AUTO, S.TILE_AUTO, 4096, 8, 0, C.byref(n), None) == 2
    assert lib.mi_matmul_mfma_timeline(C.byref(t), S.K_AUTO, S.TILE_AUTO, 4100, 8, 16, C.byref(n), None) == 2
    assert lib.mi_matmul_mfma_timeline(None, S.K_AUTO, S.TILE_AUTO, 4096, 8, 16, C.byref(n), None) == 2


def test_planner_picks_for_the_benchmark_configurations():
    p = S.matmul_mfma_plan(_t(8192, 8192, 8192, S.BF16))
    assert (p["tile"], p["k_splits"]) == ("256x256", 1)
    p = S.matmul_mfma_plan(_t(4096, 4096, 4096))
    assert (p["tile"], p["k_splits"]) == ("256x256", 1)
    p = S.matmul_mfma_plan(_t(2048, 2048, 65536))
    assert p["k_splits"] >= 2 and p["k_mode"] == "split k"          # 64 tiles of 256^2 cannot fill 256 CUs
    p = S.matmul_mfma_plan(_t(16384, 128, 8192))
    assert p["tile"] in ("64x128", "256x128", "128x128")
    p = S.matmul_mfma_plan(_t(8192, 8192, 8192), S.K_OUTPUT_STATIONARY, S.TILE_128x128)
    assert (p["tile"], p["k_splits"]) == ("128x128", 1)
    with pytest.raises(S.MiGemmError):
        S.matmul_mfma_plan(_t(100, 100, 100))


def test_planner_constants_can_be_replaced_and_read_from_the_environment():
    """The planner's two constants per tile are data: readable, replaceable for the process (what `gemm --calibrate`
    measures goes in here), and taken from MI_GEMM_PLANNER_CONSTANTS when the library is loaded.  The estimate of a
    forced plan follows them; bad values and unknown tiles are refused; a child process shows the environment path."""
    lib = S.lib()
    tile = S.TILE_256x256
    k64, fixed = S.tile_planner_constants(tile)
    assert 0.5 < k64 < 3.0 and 5.0 < fixed < 40.0
    t = _t(8192, 8192, 8192, S.BF16)
    before = S.matmul_mfma_estimate_us(t, S.K_OUTPUT_STATIONARY, tile)
    try:
        S.tile_set_planner_constants(tile, 2.0 * k64, fixed)
        assert S.tile_planner_constants(tile) == (2.0 * k64, fixed)
        assert S.matmul_mfma_estimate_us(t, S.K_OUTPUT_STATIONARY, tile) > 1.8 * before - 100.0
        # the planner now prefers another tile for the same problem
        assert S.matmul_mfma_plan(t)["tile"] != "256x256"
    finally:
        S.tile_set_planner_constants(tile, k64, fixed)
    assert S.matmul_mfma_estimate_us(t, S.K_OUTPUT_STATIONARY, tile) == pytest.approx(before)
    assert S.matmul_mfma_plan(t)["tile"] == "256x256"
    # the tile that shares its CU: the figures of a lone workgroup scale with the pair's and come back
    two = next(x["code"] for x in S.tiles() if x["workgroups_per_cu"] == 2)
    k2, f2 = S.tile_planner_constants(two)
    small = _t(192, 128, 1024)
    lone = S.matmul_mfma_estimate_us(small, S.K_OUTPUT_STATIONARY, two)
    try:
        S.tile_set_planner_constants(two, 2.0 * k2, 2.0 * f2)
        assert S.matmul_mfma_estimate_us(small, S.K_OUTPUT_STATIONARY, two) == pytest.approx(2.0 * lone, rel=0.02)
    finally:
        S.tile_set_planner_constants(two, k2, f2)
    assert S.matmul_mfma_estimate_us(small, S.K_OUTPUT_STATIONARY, two) == pytest.approx(lone)
    for bad in ((0, 1.0, 1.0), (S.tile_count(), 1.0, 1.0), (tile, 0.0, 1.0), (tile, 1.0, -1.0), (tile, float("nan"), 1.0),
                (tile, 1.0, 1e4)):
        assert lib.mi_tile_set_planner_constants(*bad) == 2
    assert lib.mi_tile_planner_constants(0, None, None) == 2 and lib.mi_tile_planner_constants(tile, None, None) == 0
    code = ("import spork_amd as S; print(S.tile_planner_constants(S.TILE_256x256), S.tile_planner_constants(S.TILE_64x128), "
            "S.tile_planner_constants(S.TILE_128x128))")
    env = dict(os.environ, MI_GEMM_PLANNER_CONSTANTS="256x256=1.5/20.5, 64x128=0.3/5,7x7=1/1,128x128=oops")
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, capture_output=True, text=True, check=True)
    assert out.stdout.strip() == f"(1.5, 20.5) (0.3, 5.0) {S.tile_planner_constants(S.TILE_128x128)}", out.stdout
    assert "skipped '7x7=1/1'" in out.stderr and "skipped '128x128=oops'" in out.stderr


def test_host_driver_is_built_against_the_abi_only():
    exe = os.path.join(ROOT, "spork_amd", "csrc", "gemm")
    assert os.path.exists(exe), "run __graft_entry__.build()"
    needed = subprocess.run(["readelf", "-d", exe], capture_output=True, text=True, check=True).stdout
    assert "libmi_gemm.so" in needed
    assert "libamdhip64" not in needed  # the host driver never links the HIP runtime itself
    for src in ("gemm_main.cpp", "gemm_test.cpp", "gemm_test.h", "gpu_tensor.h"):
        text = open(os.path.join(ROOT, "spork_amd", "csrc", src)).read()
        assert "hip/hip_runtime" not in text


def test_product_never_touches_the_oracle():
    pat = re.compile(r"^\s*(import\s+oracle|from\s+oracle\b)|liboracle|oracle/", re.M)
    for base, _, files in os.walk(os.path.join(ROOT, "spork_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp", "Makefile")):
                assert not pat.search(open(os.path.join(base, f)).read()), f
    # bench.py may use it only inside the cpu_baseline leg
    text = open(os.path.join(ROOT, "bench.py")).read()
    head, _, tail = text.partition("def cpu_baseline(")
    assert not pat.search(head)
    assert "import oracle" in tail
