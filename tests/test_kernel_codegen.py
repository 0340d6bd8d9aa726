"""Guards on the code hipcc generates for the hot kernel (CPU only: hipcc cross-compiles gfx950 without a GPU).

The kernel counts its own LDS reads with `s_waitcnt lgkmcnt(n)`, n > 0.  That counter is shared with scalar memory
loads, which return out of order.  A scalar load in flight next to the fragment reads cannot make such a wait pass too
early (with one more operation outstanding, "at most n outstanding" takes one more completion, and the fragment reads
complete in order), but it makes it wait for the scalar load as well.  So the scalar loads of the kernel's start must all
have been waited for before the first fragment read, and no K loop may contain one.
And the accumulators must stay in registers: a build whose plain (non-EDGE) kernels need scratch memory is a
performance bug the tests would not otherwise see.  And no store of more than 8 bytes per lane may have its data
registers written again within the next two instruction slots: the compiler does not insert those slots before the
moves between accumulation registers, and the GPU then stores a half-overwritten value now and then.

Every check runs over every tile's translation unit (all 18 `gemm_mfma_inst_*.hip`), read from the device assembly that the
build keeps in `spork_amd/csrc/listings/`; a unit whose listing is missing or older than its sources is compiled here."""
import glob
import os
import re
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "spork_amd", "csrc")
# every tile's translation unit: the build keeps each one's device assembly in csrc/listings/, which is what is read here
UNITS = sorted(os.path.basename(p) for p in glob.glob(os.path.join(CSRC, "gemm_mfma_inst_*.hip")))
DEEP_UNITS = [u for u in UNITS if "k32" not in u]
# tiles whose K loop has the MFMA gaps to carry hand-placed DMA halves (`LATE` in the kernel): every 64-deep tile but the two
# smallest; value: DMA instructions per wave and K tile, (BM + BN) / 32
HAND_PLACED = {u: (int(m.group(1)) + int(m.group(2))) // 32 for u in DEEP_UNITS
               if (m := re.search(r"inst_(\d+)x(\d+)\.hip", u)) and (m.group(1), m.group(2)) not in (("64", "128"), ("96", "128"))}
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-munsafe-fp-atomics", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-S", "--cuda-device-only"]
SOURCES = ["gemm_mfma_kernel.hpp", "gemm_mfma_launch.hpp", "mi_internal.hpp", os.path.join("..", "..", "include", "mi_gemm.h")]


def _listing(unit):
    """The unit's device assembly: the listing the build left (if no source is newer than it), else compiled now."""
    kept = os.path.join(CSRC, "listings", unit.replace(".hip", ".s"))
    deps = [os.path.join(CSRC, unit)] + [os.path.join(CSRC, d) for d in SOURCES]
    if os.path.exists(kept) and all(os.path.getmtime(kept) >= os.path.getmtime(d) for d in deps):
        return open(kept).read()
    if not shutil.which("hipcc"):
        return None
    out = os.path.join(tempfile.mkdtemp(prefix="codegen_"), unit + ".s")
    r = subprocess.run(["hipcc", *FLAGS, os.path.join(CSRC, unit), "-o", out], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return open(out).read()


@pytest.fixture(scope="module")
def compiled():
    assert len(UNITS) == 18 and len(HAND_PLACED) == 11, UNITS
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 2)) as pool:
        listings = dict(zip(UNITS, pool.map(_listing, UNITS)))
    if any(v is None for v in listings.values()):
        pytest.skip("no listings from the build and no hipcc on PATH")
    return listings


def _kernels(asm, with_trailer=False):
    parts = re.split(r"\n(?=_ZN7mi_gemm14gemm_tn_kernel[^\n]*:\s)", asm)
    for fn in parts[1:]:
        lines = fn.split("\n")
        end = next((i for i, l in enumerate(lines) if "s_endpgm" in l), len(lines))
        if with_trailer:
            yield lines[0].split(":")[0], lines[:end], lines[end:]
        else:
            yield lines[0].split(":")[0], lines[:end]


def _is_range_checked(name):
    # last template arguments: ATOMIC either way, EDGE, not stream-K, ordinary loads
    return name.endswith("Lb1ELb0ELi0EEEvNS_8GemmArgsE")


@pytest.mark.parametrize("unit", UNITS)
def test_no_scalar_load_shares_the_counter_with_fragment_reads(compiled, unit):
    asm = compiled[unit]
    seen = 0
    for name, lines in _kernels(asm):
        seen += 1
        reads = [i for i, l in enumerate(lines) if "ds_read_b128" in l]
        first_read = reads[0]
        scalar_loads = [i for i, l in enumerate(lines) if re.search(r"\bs_(load|buffer_load)_", l)]
        early = [i for i in scalar_loads if i < first_read]
        assert early, name
        assert any("lgkmcnt(0)" in l for l in lines[max(early):first_read]), name
        # Later ones (kernel arguments that only the code behind the K loop needs, which the compiler loads where it runs
        # out of scalar registers) must not sit inside a K loop: a loop that reads fragments and stores nothing
        labels = {m.group(1): i for i, l in enumerate(lines) if (m := re.match(r"(\.LBB\d+_\d+):", l))}
        for j, l in enumerate(lines):
            m = re.match(r"\s+s_cbranch_\w+ (\.LBB\d+_\d+)", l)
            if m and labels.get(m.group(1), j) < j:
                body = lines[labels[m.group(1)]:j]
                if any("ds_read_b128" in x for x in body) and not any(re.search(r"\b(buffer|global)_(store|atomic)", x) for x in body):
                    assert not any(re.search(r"\bs_(load|buffer_load)_", x) for x in body), (name, m.group(1))
    # two dtypes x ({plain, atomic} x {plain, range-checked}, plus the stream-K build and the two non-temporal twins
    # of the plain and of the atomic whole-tile build of the 64-deep tiles)
    assert seen == (18 if "k32" not in unit else 8)


@pytest.mark.parametrize("unit", DEEP_UNITS)
def test_non_temporal_builds_mark_exactly_one_operand(compiled, unit):
    """The builds for an operand that is read once set the `nt` bit on that operand's DMA only: half of the DMA
    instructions of the 256x256 tile (A and B tiles are the same size), and none in any other build."""
    asm = compiled[unit]
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
    """Scratch bytes per lane as the assembler records them behind each kernel: none in any whole-tile build of any tile;
    the range-checked builds of the largest tiles may spill a few registers.  And the one tile that shares a CU between two
    workgroups must leave room for two waves per SIMD."""
    asm = compiled[unit]
    seen = 0
    for name, _, trailer in _kernels(asm, with_trailer=True):
        text = "\n".join(trailer)
        size = int(re.search(r"; ScratchSize: (\d+)", text).group(1))
        seen += 1
        if not _is_range_checked(name):
            assert size == 0, (name, size)
        else:
            assert size <= 64, (name, size)
        if "192x128" in unit:
            assert int(re.search(r"; Occupancy: (\d+)", text).group(1)) >= 2, name
    assert seen == (18 if "k32" not in unit else 8)


def _registers(token):
    m = re.match(r"([av])\[(\d+):(\d+)\]$", token)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"([av])(\d+)$", token)
    return {(m.group(1), int(m.group(2)))} if m else set()


@pytest.mark.parametrize("unit", UNITS)
def test_wide_store_data_is_not_overwritten_in_the_next_two_slots(compiled, unit):
    asm = compiled[unit]
    stores = 0
    for name, lines in _kernels(asm):
        code = [l.strip() for l in lines if l.startswith("\t") and not l.strip().startswith((";", "."))]
        for i, line in enumerate(code):
            if not re.match(r"(buffer|global)_store_dwordx[34]\b", line):
                continue
            stores += 1
            # (buffer stores name their data first, global stores their address)
            operands = [o.strip() for o in line.split(None, 1)[1].split(",")]
            data = _registers(operands[1] if line.startswith("global_") else operands[0])
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


@pytest.mark.parametrize("unit", sorted(HAND_PLACED))
def test_hand_placed_dma_finds_its_lds_base_in_m0(compiled, unit):
    """The K loops of the larger tiles issue their DMAs through inline assembly: `s_mov_b32 m0, <LDS base>` in one MFMA gap,
    the `buffer_load_dwordx4 ... lds` that reads M0 in the next (`s_add_i32 m0, <base>, <constant>` for all but the first).  The compiler does not know M0 is live in between, so
    nothing else may write M0 there: in the steady loop of every whole-tile build each DMA must be preceded by exactly
    one write of M0 since the DMA before it, that write must be the hand-placed move, and an MFMA (the wait state the
    write needs) must lie between the two."""
    asm = compiled[unit]
    dmas_per_k_tile = HAND_PLACED[unit]
    checked = 0
    for name, lines in _kernels(asm):
        if _is_range_checked(name):  # range-checked builds keep the compiler's own DMA
            continue
        loops = [b for b in _branch_free_loops(lines) if sum(x.startswith("v_mfma") for x in b) >= 16]  # (not the loops of the sum)
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
                    assert "lds" in l.split(";")[0].split(), l
                    dmas += 1
                    assert len(writes) == 1 and re.match(r"s_(mov_b32 m0, s\d+|add_i32 m0, s\d+, 0x[0-9a-f]+) ; dma-base$", writes[0]), (name[-40:], writes)
                    assert mfma_since_write >= 1, name[-40:]
                    writes = []
            assert dmas == dmas_per_k_tile, (name[-40:], dmas)
            checked += 1
    assert checked >= 10


@pytest.mark.parametrize("unit", UNITS)
def test_no_other_write_of_m0_between_the_halves_of_a_hand_placed_dma(compiled, unit):
    """The same rule for every block of every kernel of every tile, steady or not (the first and last iterations of a K
    loop run the hand-placed halves under run-time flags): reading the listing top to bottom, the last instruction that
    wrote M0 before a hand-placed DMA (marked `dma-issue` by the kernel source) must be a hand-placed base (marked
    `dma-base`), with at least one MFMA or wait state between the two.  A write of M0 that the compiler put between the
    halves - for an LDS DMA of its own, say - would be found here as the last writer."""
    asm = compiled[unit]
    issues = 0
    for name, lines in _kernels(asm):
        code = [l.strip() for l in lines if l.startswith("\t") and not l.strip().startswith((";", "."))]
        last_write, states = None, 0
        for l in code:
            op = l.split()[0]
            if op.startswith("s_") and re.match(r"m0\b", l[len(op):].strip()):
                last_write, states = l, 0
            elif op.startswith("v_mfma") or op == "s_nop":
                states += 1
            if l.endswith("; dma-issue"):
                issues += 1
                assert last_write is not None and last_write.endswith("; dma-base"), (name[-40:], last_write, l)
                assert states >= 1, (name[-40:], last_write, l)
        if unit in HAND_PLACED and not _is_range_checked(name):
            assert sum(l.endswith("; dma-issue") for l in code) >= HAND_PLACED[unit], name[-40:]
    assert (issues > 0) == (unit in HAND_PLACED), (unit, issues)
