"""BASELINE configs[0] as it is stated: fp16 512^3, entries uniform[-1,1] from seed, A row-major M x K, B stored N x K,
fp32 accumulate and fp32 C, "run through the reference CPU GEMM (plumbing, no GPU needed)".

The reference CPU GEMM is the Exo proc nyc25_gemm_cpu (docs/nyc25.py:16-55: for m / for n / accum: f32 = 0 / for k:
accum += A[m,k] * B[k,n] / C[m,n] = accum) with B indexed [n,k] as in xgemm_Sm80.py:334-336.  The oracle's port of it
(orc_gemm_ref_f32) runs the whole configuration here on one thread and on several, and is held against the fp64 oracle
on the same quantised inputs.  No GPU and no HIP library is touched.
"""
import os
import time

import numpy as np

M = N = K = 512
SEED_A, SEED_B = 20010106, 19980724  # the reference's constants (gemm/gemm_test.cu:76,87)


def test_c1_through_the_reference_cpu_gemm(oracle):
    f16, uniform = oracle.F16, 3
    a = oracle.fill(M, K, uniform, False, f16, 1.0, SEED_A)   # A[m,k], row-major
    b = oracle.fill(N, K, uniform, True, f16, 1.0, SEED_B)    # logical B[k,n] stored N x K (transpose rule, gemm_test.cu:64-65)
    va, vb = oracle.widen(a, f16), oracle.widen(b, f16)
    assert -1.0 <= va.min() < -0.99 and 0.99 < va.max() <= 1.0 and abs(float(va.mean())) < 0.01
    assert -1.0 <= vb.min() < -0.99 and 0.99 < vb.max() <= 1.0

    t0 = time.perf_counter()
    c1 = oracle.gemm_ref_f32(M, N, K, a, b, f16, threads=1)
    t1 = time.perf_counter()
    threads = max(2, min(oracle.max_threads(), os.cpu_count() or 2, 16))
    cn = oracle.gemm_ref_f32(M, N, K, a, b, f16, threads=threads)
    t2 = time.perf_counter()
    # OpenMP splits over m only: every element is still one sequential k loop, so the bits cannot depend on the threads
    np.testing.assert_array_equal(c1, cn)

    ref = oracle.gemm_f64(M, N, K, a, b, f16)
    absref = oracle.gemm_f64(M, N, K, a, b, f16, abs_mode=True)   # sum_k |a||b|
    err = oracle.error_metrics(c1, ref, absref)
    flop = 2.0 * M * N * K
    print(f"C1 fp16 {M}^3 through the reference CPU GEMM: 1 thread {flop / (t1 - t0) * 1e-9:.2f} GFLOP/s, "
          f"{threads} threads {flop / (t2 - t1) * 1e-9:.2f} GFLOP/s ({os.cpu_count()} cores here); "
          f"max rel err {err['max_rel_err']:.2e}, componentwise {err['max_componentwise']:.2e}")
    # the benchmark's gate (normalised max error) and the textbook bound of a length-K fp32 sum, element by element
    assert err["max_rel_err"] <= 1e-3
    bound = K * 2.0 ** -24 * absref * (1.0 + 1e-6) + 1e-30
    assert np.all(np.abs(c1.astype(np.float64) - ref) <= bound)
    assert err["max_componentwise"] <= K * 2.0 ** -24
    # the fp64 oracle is itself the exact product of the quantised inputs to fp64 rounding: numpy agrees
    np.testing.assert_allclose(ref, va.astype(np.float64) @ vb.astype(np.float64).T, rtol=0, atol=1e-9)
    # and a dropped or doubled term would show: the same check fails on a perturbed C
    bad = c1.copy()
    bad[300, 17] += np.float32(4.0 * K * 2.0 ** -24 * absref[300, 17] + 1e-3)
    assert not np.all(np.abs(bad.astype(np.float64) - ref) <= bound)
