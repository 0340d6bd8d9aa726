"""Pins the CPU oracle (test infrastructure) without the reference: golden fixtures made from Python integers and
numpy/torch routines, exhaustive number-format checks against library casts, brute force on tiny shapes, closed forms
of the reference driver's known-answer inputs, and Freivalds' identity.  Runs on the CPU."""
import functools
import json
import os

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ------------------------------------------------------------------------------------------------ pcg3d
def test_pcg3d_golden_vectors(oracle):
    vecs = json.load(open(os.path.join(GOLD, "pcg3d_vectors.json")))
    assert len(vecs) >= 30
    for v in vecs:
        assert oracle.pcg3d(v["x"], v["y"], v["z"]) == v["h"], v


def test_pcg3d_packing_structure(oracle):
    """Bits 0..11 of the packed value come from the x output alone and bits 44..55 from the z output alone (y<<12
    spans 12..43, z<<24 spans 24..55): a wrong shift or a mis-parenthesised xor breaks one of these."""
    from golden.make_golden import pcg3d_xyz

    rng = np.random.default_rng(1)
    for _ in range(200):
        x, y, z = (int(v) for v in rng.integers(0, 1 << 32, 3))
        h = oracle.pcg3d(x, y, z)
        ox, oy, oz = pcg3d_xyz(x, y, z)
        assert h < 1 << 56
        assert h & 0xFFF == ox & 0xFFF
        assert h >> 44 == oz >> 20
        assert (h >> 12) & 0xFFF == ((ox >> 12) ^ oy) & 0xFFF  # bits 12..23: x and y only
    assert oracle.pcg3d(1, 2, 3) != oracle.pcg3d(2, 1, 3)


# ---------------------------------------------------------------------------------------- number formats
def test_f16_widening_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = np.array([oracle.lib().orc_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    want = bits.view(np.float16).astype(np.float32)
    np.testing.assert_array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_bf16_widening_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = np.array([oracle.lib().orc_bf16_to_f32(int(b)) for b in bits], dtype=np.float32)
    want = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    ok = ~np.isnan(want)
    np.testing.assert_array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])


def _float_sweep():
    rng = np.random.default_rng(3)
    parts = [rng.standard_normal(20000).astype(np.float32), (rng.standard_normal(5000) * 1e-6).astype(np.float32),
             (rng.standard_normal(5000) * 3e4).astype(np.float32), rng.integers(0, 1 << 32, 30000, dtype=np.uint32).view(np.float32)]
    # every fp16 value, the midpoints between neighbours and their float neighbours (ties and near-ties)
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    parts += [h, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), -mid,
              np.array([65504, 65519.996, 65520, 65536, 1e10, 5.96e-8, 2.98e-8, 2.9802322e-08, 3e-8, 0.0, -0.0, np.inf, -np.inf],
                       dtype=np.float32)]
    x = np.concatenate(parts)
    return x[~np.isnan(x)]


def test_f16_narrowing_matches_numpy_rne(oracle):
    x = _float_sweep()
    L = oracle.lib()
    got = np.array([L.orc_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got, want)


def test_bf16_narrowing_matches_torch_rne(oracle):
    x = _float_sweep()
    L = oracle.lib()
    got = np.array([L.orc_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)


# --------------------------------------------------------------------------------------------- generators
def test_identity_and_tiled_numbers_closed_forms(oracle):
    for dtype, mod, stride in ((oracle.F16, 32, 64), (oracle.BF16, 16, 16)):
        for tr in (False, True):
            ident = oracle.widen(oracle.fill(70, 90, oracle.IDENTITY, tr, dtype), dtype)
            np.testing.assert_array_equal(ident, np.eye(70, 90, dtype=np.float32))
            t = oracle.widen(oracle.fill(70, 90, oracle.TILED_NUMBERS, tr, dtype), dtype)
            r, c = np.meshgrid(np.arange(70), np.arange(90), indexing="ij")
            x, y = (r, c) if tr else (c, r)
            np.testing.assert_array_equal(t, ((x % mod) + stride * (y % mod)).astype(np.float32))
            assert t.max() <= (2047 if dtype == oracle.F16 else 255)  # exactly representable


def test_uniform_is_exact_and_in_range(oracle):
    """u = low 24 bits of the hash / 2^24, value = a (2u - 1): every step is exact in fp32."""
    for a in (1.0, 0.5):
        bits = oracle.fill(64, 64, oracle.UNIFORM, False, oracle.F16, a, 4242)
        vals = oracle.widen(bits, oracle.F16)
        assert vals.min() >= -a and vals.max() <= a
        for (r, c) in [(0, 0), (5, 9), (63, 63)]:
            h = oracle.pcg3d(c, r, 4242)
            v = np.float32(a) * np.float32((h & 0xFFFFFF) * 2.0 - 2 ** 24) / np.float32(2 ** 24)
            assert vals[r, c] == np.float32(v).astype(np.float16).astype(np.float32)
    # transpose_rule stores the same logical matrix transposed (gemm/gemm_test.cu:64-65,241)
    direct = oracle.fill(30, 50, oracle.UNIFORM, False, oracle.F16, 1.0, 99)
    transposed = oracle.fill(50, 30, oracle.UNIFORM, True, oracle.F16, 1.0, 99)
    np.testing.assert_array_equal(direct, transposed.T)


def test_normal_is_box_muller_of_the_hash(oracle):
    K = 4096
    scale = K ** -0.5
    bits = oracle.fill(256, 256, oracle.NORMAL, False, oracle.BF16, scale, 20010106)
    vals = oracle.widen(bits, oracle.BF16).astype(np.float64) / scale
    assert abs(vals.mean()) < 0.02 and abs(vals.std() - 1.0) < 0.02
    assert abs((np.abs(vals) < 1).mean() - 0.6827) < 0.01
    for (r, c) in [(0, 0), (17, 3), (255, 254)]:
        h1 = oracle.pcg3d(c, r, 20010106)
        h2 = oracle.pcg3d(c, r, 20010106 ^ 0x9E3779B9)
        u1 = ((h1 & 0xFFFFFF) + 1) / 2 ** 24
        u2 = (h2 & 0xFFFFFF) / 2 ** 24
        v = np.sqrt(-2 * np.log(u1)) * np.cos(2 * np.pi * u2) * scale
        want = torch.tensor(np.float32(v)).to(torch.bfloat16).to(torch.float32).item()
        assert oracle.widen(bits, oracle.BF16)[r, c] == pytest.approx(want, rel=2 ** -7)


def test_reference_random_style_statistics(oracle):
    """gemm/gemm_test.cu:73-91: 75 % zeros, 25 % u^4 in [0,1), a 1-in-100000 spike of 1000, never negative."""
    v = oracle.widen(oracle.fill(1024, 1024, oracle.RANDOM, False, oracle.F16), oracle.F16)
    assert v.min() >= 0
    assert abs((v == 0).mean() - 0.75) < 0.02  # u^4 underflows to 0 in fp16 for a few more
    spikes = (v == 1000).sum()
    assert 0 < spikes < 40
    rest = v[(v != 0) & (v != 1000)]
    assert rest.max() <= 1.0


def test_reference_random_style_hand_evaluated_elements(oracle):
    """Elements of the sparse random style worked out from Python integers and numpy float32 arithmetic
    (tests/golden/make_golden.py): zeros, fourth powers and every spike of 1000 in the first 1024 x 1024 coordinates.
    A wrong modulus, a wrong seed or v^2 for v^4 changes these bits."""
    vecs = json.load(open(os.path.join(GOLD, "random_style_vectors.json")))
    kinds = {v["kind"] for v in vecs}
    assert kinds == {"zero", "fourth_power", "spike"} and len(vecs) >= 28
    plain = {d: oracle.fill(1024, 1024, oracle.RANDOM, False, d) for d in (oracle.F16, oracle.BF16)}
    swapped = {d: oracle.fill(1024, 1024, oracle.RANDOM, True, d) for d in (oracle.F16, oracle.BF16)}
    for v in vecs:
        x, y = v["x"], v["y"]
        f32 = np.float32(oracle.element(y, x, oracle.RANDOM, False, oracle.F16))
        assert int(f32.view(np.uint32)) == v["f32_bits"], v
        for d, key in ((oracle.F16, "f16_bits"), (oracle.BF16, "bf16_bits")):
            assert int(plain[d][y, x]) == v[key], v        # x is the column
            assert int(swapped[d][x, y]) == v[key], v      # transpose rule: x is the row
    # the fixture holds every spike of that range: the oracle has no other
    spikes = {(v["x"], v["y"]) for v in vecs if v["kind"] == "spike"}
    ys, xs = np.nonzero(oracle.widen(plain[oracle.F16], oracle.F16) == 1000)
    assert {(int(x), int(y)) for x, y in zip(xs, ys)} == spikes


# ------------------------------------------------------------------------------------------------- GEMMs
@pytest.mark.parametrize("name,dtype", [("f16", 0), ("bf16", 1)])
@pytest.mark.parametrize("a_col", [0, 1])
@pytest.mark.parametrize("b_col", [0, 1])
def test_gemm_f64_matches_numpy_golden_in_every_layout(oracle, name, dtype, a_col, b_col):
    g = np.load(os.path.join(GOLD, "gemm_small.npz"))
    M, N, K = 48, 40, 80
    a = g[f"{name}_a_{'colmajor' if a_col else 'rowmajor'}"]
    b = g[f"{name}_b_{'colmajor' if b_col else 'rowmajor'}"]
    want = g[f"{name}_c_f64"]
    for fn in (oracle.gemm_f64, oracle.gemm_f64_naive):
        got = fn(M, N, K, a, b, dtype, a_col, b_col)
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-12)
    np.testing.assert_allclose(oracle.gemm_f64(M, N, K, a, b, dtype, a_col, b_col, abs_mode=True), g[f"{name}_abs_c_f64"], atol=1e-12)
    rows = np.array([0, 7, 47, 13], dtype=np.uint32)
    np.testing.assert_allclose(oracle.gemm_f64_rows(M, N, K, a, b, dtype, rows, a_col, b_col), want[rows], atol=1e-12)
    cols = np.array([39, 0, 5], dtype=np.uint32)
    np.testing.assert_allclose(oracle.gemm_f64_cols(M, N, K, a, b, dtype, cols, a_col, b_col), want[:, cols], atol=1e-12)


def test_blocked_equals_brute_force_on_ragged_shapes(oracle):
    rng = np.random.default_rng(11)
    for (M, N, K) in [(1, 1, 1), (3, 5, 7), (65, 9, 1030), (130, 67, 2049)]:
        a = rng.integers(0, 1 << 16, (M, K), dtype=np.uint16) & np.uint16(0xBBFF)  # finite fp16 values below 2
        b = rng.integers(0, 1 << 16, (N, K), dtype=np.uint16) & np.uint16(0xBBFF)
        np.testing.assert_allclose(oracle.gemm_f64(M, N, K, a, b, 0), oracle.gemm_f64_naive(M, N, K, a, b, 0), rtol=1e-13, atol=1e-13)


def test_reference_cpu_gemm_is_sequential_fp32(oracle):
    """The reference CPU GEMM accumulates in fp32 in k order (docs/nyc25.py:43-52): reproduce that with numpy scalars."""
    g = np.load(os.path.join(GOLD, "gemm_small.npz"))
    M, N, K = 48, 40, 80
    for name, dtype in (("f16", 0), ("bf16", 1)):
        a, b = g[f"{name}_a_rowmajor"], g[f"{name}_b_colmajor"]
        aw, bw = oracle.widen(a, dtype), oracle.widen(b, dtype)
        got = oracle.gemm_ref_f32(M, N, K, a, b, dtype)
        got_mt = oracle.gemm_ref_f32(M, N, K, a, b, dtype, threads=4)
        np.testing.assert_array_equal(got, got_mt)
        for (m, n) in [(0, 0), (47, 39), (20, 7), (3, 31)]:
            prods = aw[m] * bw[n]  # exact in fp32
            want = functools.reduce(lambda s, p: np.float32(s + p), prods, np.float32(0))
            assert got[m, n] == want
        # every layout flag combination gives the same C
        for ac in (0, 1):
            for bc in (0, 1):
                for cc in (0, 1):
                    aa = g[f"{name}_a_{'colmajor' if ac else 'rowmajor'}"]
                    bb = g[f"{name}_b_{'colmajor' if bc else 'rowmajor'}"]
                    c = oracle.gemm_ref_f32(M, N, K, aa, bb, dtype, ac, bc, cc)
                    np.testing.assert_array_equal(c.T if cc else c, got)
        # partial row range leaves other rows untouched
        part = oracle.gemm_ref_f32(M, N, K, a, b, dtype, m_begin=8, m_end=16)
        np.testing.assert_array_equal(part[8:16], got[8:16])
        assert not part[:8].any() and not part[16:].any()


def test_known_answers_of_the_reference_driver(oracle):
    """gemm/gemm_main.cpp:81-90: tiled x identity gives C = A[:, :N]; identity x tiled gives C = B[:M, :]."""
    M, N, K = 96, 64, 128
    for dtype in (0, 1):
        a = oracle.fill(M, K, oracle.TILED_NUMBERS, False, dtype)
        b = oracle.fill(N, K, oracle.IDENTITY, True, dtype)
        np.testing.assert_array_equal(oracle.gemm_f64(M, N, K, a, b, dtype), oracle.widen(a, dtype)[:, :N].astype(np.float64))
        np.testing.assert_array_equal(oracle.gemm_ref_f32(M, N, K, a, b, dtype), oracle.widen(a, dtype)[:, :N])
        a = oracle.fill(M, K, oracle.IDENTITY, False, dtype)
        b = oracle.fill(N, K, oracle.TILED_NUMBERS, True, dtype)
        np.testing.assert_array_equal(oracle.gemm_f64(M, N, K, a, b, dtype), oracle.widen(b, dtype).T[:M, :].astype(np.float64))


# --------------------------------------------------------------------------------- checks and statistics
def test_freivalds_accepts_truth_and_catches_one_wrong_element(oracle):
    M, N, K = 96, 80, 256
    a = oracle.fill(M, K, oracle.UNIFORM, False, 0, 1.0, 1)
    b = oracle.fill(N, K, oracle.UNIFORM, True, 0, 1.0, 2)
    c = oracle.gemm_f64(M, N, K, a, b, 0).astype(np.float32)
    resid, scale = oracle.freivalds(M, N, K, a, b, c, 0)
    assert (resid / scale).max() < 1e-6
    bad = c.copy()
    bad[17, 33] += 0.5
    resid, scale = oracle.freivalds(M, N, K, a, b, bad, 0)
    assert resid.min() > 0.49  # every +-1 vector sees the full perturbation
    bad = c.copy()
    bad[5, 5] = np.nan
    assert np.isinf(oracle.freivalds(M, N, K, a, b, bad, 0)[0]).all()
    # column-major C is read through its flag
    resid, scale = oracle.freivalds(M, N, K, a, b, np.ascontiguousarray(c.T), 0, c_col_major=1)
    assert (resid / scale).max() < 1e-6


def test_error_metrics(oracle):
    ref = np.arange(12, dtype=np.float64).reshape(3, 4)
    c = ref.astype(np.float32).copy()
    c[2, 1] += 0.25
    m = oracle.error_metrics(c, ref, np.full((3, 4), 10.0))
    assert m["max_abs_err"] == 0.25 and m["worst"] == (2, 1) and m["max_abs_ref"] == 11.0
    assert m["max_rel_err"] == pytest.approx(0.25 / 11) and m["max_componentwise"] == pytest.approx(0.025)
    assert np.isinf(oracle.error_metrics(np.full((3, 4), np.nan, np.float32), ref)["max_abs_err"])


def test_compare_rule_of_the_reference(oracle):
    """gemm/gemm_test.cu:138-147."""
    one = np.ones((2, 3), dtype=np.float32)
    assert oracle.compare_ratio(one, one) is None
    assert oracle.compare_ratio(np.zeros((2, 3), np.float32), np.zeros((2, 3), np.float32)) is None
    y = one.copy(); y[1, 2] = 1.03
    assert oracle.compare_ratio(one, y) is None          # 1.03 < 1 + 1/32
    y[1, 2] = 1.04
    assert oracle.compare_ratio(one, y) == (1, 2)        # 1.04 > 1.03125
    y = one.copy(); y[0, 1] = -1
    assert oracle.compare_ratio(one, y) == (0, 1)        # sign
    y = one.copy(); y[1, 0] = 0
    assert oracle.compare_ratio(one, y) == (1, 0)        # one side zero: ratio is inf
    y = one.copy(); y[0, 0] = np.nan; y[1, 1] = 5
    assert oracle.compare_ratio(one, y) == (0, 0)        # first failure in row-major order
    poison = np.full((2, 3), np.frombuffer(b"\x7d\x7d\x7d\x7d", np.float32)[0])
    assert oracle.compare_ratio(one, poison) == (0, 0)   # an unwritten (0x7D-poisoned) element fails


def test_iqr_mean_is_mean_of_sorted_samples_6_to_18(oracle):
    """gemm/gemm_test.cu:399-404 with 25 samples: indices 6..18 of the sorted times."""
    t = np.arange(25, dtype=np.float32)[::-1].copy()
    t[0] = 1000.0  # outlier lands outside the window
    assert oracle.iqr_mean(t) == pytest.approx(np.sort(t)[6:19].mean())
    assert oracle.iqr_mean(np.array([3.0], np.float32)) == 3.0
