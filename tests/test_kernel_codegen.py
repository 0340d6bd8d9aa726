"""Guards on the code hipcc generates for the hot kernel (CPU only: hipcc cross-compiles gfx950 without a GPU).

The kernel counts its own LDS reads with `s_waitcnt lgkmcnt(n)`, n > 0.  That counter is shared with scalar memory
loads, which return out of order: one scalar load in flight next to the fragment reads would make the partial waits
meaningless, silently.  So every scalar load must sit before the first fragment read, with a full wait in between.
And the accumulators must stay in registers: a build whose plain (non-EDGE) kernels need scratch memory is a
performance bug the tests would not otherwise see.  And no store of more than 8 bytes per lane may have its data
registers written again within the next two instruction slots: the compiler does not insert those slots before the
moves between accumulation registers, and the GPU then stores a half-overwritten value now and then."""
import os
import re
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "spork_amd", "csrc")
UNITS = ["gemm_mfma_inst_256x256.hip", "gemm_mfma_inst_64x128k32.hip",  # the flagship tile and a 32x32x16 twin
         "gemm_mfma_inst_192x128.hip"]  # the tile of which two workgroups share a CU
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-munsafe-fp-atomics", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-S", "--cuda-device-only",
         "-Rpass-analysis=kernel-resource-usage"]


def _compile(unit):
    out = os.path.join(tempfile.mkdtemp(prefix="codegen_"), unit + ".s")
    r = subprocess.run(["hipcc", *FLAGS, os.path.join(CSRC, unit), "-o", out], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return open(out).read(), r.stderr


@pytest.fixture(scope="module")
def compiled():
    if not shutil.which("hipcc"):
        pytest.skip("hipcc not on PATH")
    with ThreadPoolExecutor(max_workers=len(UNITS)) as pool:
        return dict(zip(UNITS, pool.map(_compile, UNITS)))


def _kernels(asm):
    parts = re.split(r"\n(?=_ZN7mi_gemm14gemm_tn_kernel[^\n]*:\s)", asm)
    for fn in parts[1:]:
        lines = fn.split("\n")
        end = next((i for i, l in enumerate(lines) if "s_endpgm" in l), len(lines))
        yield lines[0].split(":")[0], lines[:end]


@pytest.mark.parametrize("unit", UNITS)
def test_no_scalar_load_shares_the_counter_with_fragment_reads(compiled, unit):
    asm, _ = compiled[unit]
    seen = 0
    for name, lines in _kernels(asm):
        seen += 1
        first_read = next(i for i, l in enumerate(lines) if "ds_read_b128" in l)
        scalar_loads = [i for i, l in enumerate(lines) if re.search(r"\bs_(load|buffer_load)_", l)]
        assert scalar_loads and max(scalar_loads) < first_read, name
        between = lines[max(scalar_loads):first_read]
        assert any("lgkmcnt(0)" in l for l in between), name
    # two dtypes x ({plain, atomic} x {plain, range-checked}, plus the stream-K build and the two non-temporal twins
    # of the plain and of the atomic whole-tile build of the 64-deep tiles)
    assert seen == (18 if "k32" not in unit else 8)


@pytest.mark.parametrize("unit", [u for u in UNITS if "k32" not in u])
def test_non_temporal_builds_mark_exactly_one_operand(compiled, unit):
    """The builds for an operand that is read once set the `nt` bit on that operand's DMA only: half of the DMA
    instructions of the 256x256 tile (A and B tiles are the same size), and none in any other build."""
    asm, _ = compiled[unit]
    counts = {}
    for name, lines in _kernels(asm):
        dma = [l for l in lines if re.search(r"\bbuffer_load_dwordx4\b.*\blds\b", l)]
        assert dma, name
        once = int(re.search(r"Li(\d)EEEvNS_8GemmArgsE$", name).group(1))
        counts[name] = (once, sum(1 for l in dma if re.search(r"\bnt\b", l)), len(dma))
    assert sorted(o for o, _, _ in counts.values()) == [0] * 10 + [1] * 4 + [2] * 4
    for name, (once, marked, total) in counts.items():
        if once == 0:
            assert marked == 0, name
        else:
            assert 0 < marked < total, (name, marked, total)
            if "256x256" in unit:
                assert 2 * marked == total, (name, marked, total)


@pytest.mark.parametrize("unit", UNITS)
def test_plain_kernels_keep_everything_in_registers(compiled, unit):
    _, remarks = compiled[unit]
    names = re.findall(r"Function Name: (\S+)", remarks)
    scratch = [int(x) for x in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", remarks)]
    assert len(names) == len(scratch) == (18 if "k32" not in unit else 8)
    for name, size in zip(names, scratch):
        edge = name.endswith("Lb1ELb0ELi0EEEvNS_8GemmArgsE")  # last template arguments: range-checked, not stream-K, ordinary loads
        if not edge:
            assert size == 0, (name, size)
        else:
            assert size <= 64, (name, size)


def _registers(token):
    m = re.match(r"([av])\[(\d+):(\d+)\]$", token)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"([av])(\d+)$", token)
    return {(m.group(1), int(m.group(2)))} if m else set()


@pytest.mark.parametrize("unit", UNITS)
def test_wide_store_data_is_not_overwritten_in_the_next_two_slots(compiled, unit):
    asm, _ = compiled[unit]
    stores = 0
    for name, lines in _kernels(asm):
        code = [l.strip() for l in lines if l.startswith("\t") and not l.strip().startswith((";", "."))]
        for i, line in enumerate(code):
            if not re.match(r"(buffer|global)_store_dwordx[34]\b", line):
                continue
            stores += 1
            data = _registers(line.split()[1].rstrip(","))
            assert data, line
            slots = 0
            for nxt in code[i + 1:i + 4]:
                op, _, rest = nxt.partition(" ")
                if op == "s_nop":
                    slots += int(rest.strip()) + 1
                    continue
                if slots >= 2:
                    break
                written = _registers(rest.split(",")[0].strip()) if op.startswith(("v_", "ds_read", "buffer_load", "global_load")) else set()
                assert not (written & data), (name[-40:], line, nxt)
                slots += 1
    assert stores > 100 or "k32" in unit  # (the 32x32x16 twins store one dword per lane)


def _branch_free_loops(lines):
    """Bodies of the loops (label ... backward branch to it) that contain no other branch: the steady K loops."""
    labels = {m.group(1): i for i, l in enumerate(lines) if (m := re.match(r"(\.LBB\d+_\d+):", l))}
    for i, l in enumerate(lines):
        m = re.match(r"\s+s_cbranch_\w+ (\.LBB\d+_\d+)", l)
        if m and labels.get(m.group(1), i) < i:
            body = [x.strip() for x in lines[labels[m.group(1)] + 1:i] if x.startswith("\t") and not x.strip().startswith((";", "."))]
            if not any(x.startswith(("s_cbranch", "s_branch")) for x in body):
                yield body


@pytest.mark.parametrize("unit,dmas_per_k_tile", [("gemm_mfma_inst_256x256.hip", 16), ("gemm_mfma_inst_192x128.hip", 10)])
def test_hand_placed_dma_finds_its_lds_base_in_m0(compiled, unit, dmas_per_k_tile):
    """The K loops of the larger tiles issue their DMAs through inline assembly: `s_mov_b32 m0, <LDS base>` in one MFMA gap,
    the `buffer_load_dwordx4 ... lds` that reads M0 in the next (`s_add_i32 m0, <base>, <constant>` for all but the first).  The compiler does not know M0 is live in between, so
    nothing else may write M0 there: in the steady loop of every whole-tile build each DMA must be preceded by exactly
    one write of M0 since the DMA before it, that write must be the hand-placed move, and an MFMA (the wait state the
    write needs) must lie between the two.  (The general iterations at either end of the K loop run the same source with
    the DMAs under run-time flags; their branches make a linear reading of the listing meaningless.)"""
    asm, _ = compiled[unit]
    checked = 0
    for name, lines in _kernels(asm):
        if "Lb1ELb0ELi0EEEvNS_8GemmArgsE" in name:  # range-checked builds keep the compiler's own DMA
            continue
        loops = [b for b in _branch_free_loops(lines) if sum(x.startswith("v_mfma") for x in b) >= 48]
        assert loops, name[-40:]
        for body in loops:
            # (the loop is a cycle: start reading at its first DMA so that the write ahead of it is seen at the end)
            first = next(i for i, l in enumerate(body) if l.startswith("buffer_load_dwordx4"))
            body = body[first + 1:] + body[:first + 1]
            writes, mfma_since_write, dmas = [], 0, 0
            for l in body:
                op = l.split()[0]
                if op.startswith("s_") and re.search(r"\bm0\b", l.split(",")[0]):
                    writes.append(l)
                    mfma_since_write = 0
                elif op.startswith("v_mfma"):
                    mfma_since_write += 1
                elif op == "buffer_load_dwordx4":
                    assert l.rstrip().endswith("lds"), l
                    dmas += 1
                    assert len(writes) == 1 and re.match(r"s_(mov_b32 m0, s\d+|add_i32 m0, s\d+, 0x[0-9a-f]+)$", writes[0]), (name[-40:], writes)
                    assert mfma_since_write >= 1, name[-40:]
                    writes = []
            assert dmas == dmas_per_k_tile, (name[-40:], dmas)
            checked += 1
    assert checked >= 10
