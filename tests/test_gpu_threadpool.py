"""The library driven by the reference's real caller: the thread pool of
src/ck_threadpool.c dispatching version/v7/src/ck_parallel_decode.c's work
functions, which call the *_parallel_simd kernels concurrently from every pool
thread with (ith, nth) (ck_parallel_decode.c:112-125, 174-260).  Both pool
sizes and both CKQ_PARALLEL_MODE settings give the serial call's bits."""
import importlib
import sys

import numpy as np
import pytest

import ckq_testlib as T

pytestmark = pytest.mark.gpu

ckq = importlib.import_module("c-kernel-engine_amd")
P = ckq.parity


def say(*a):
    print(*a)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def pool():
    import torch
    assert torch.cuda.is_available()
    L = ckq.lib()
    assert L.ckq_init() == 0
    p = T.ref_pool(ckq.lib_path())
    if p is None:
        pytest.skip("oracle/_ref/libckref_pool.so has not been built (needs the reference checkout at build time)")
    yield p
    p.ck_threadpool_global_destroy()
    L.ckq_set_parallel_whole(-1)
    L.ckq_weights_clear()


@pytest.mark.parametrize("threads", [8, 16])
@pytest.mark.parametrize("whole", [0, 1])
def test_parallel_dispatch_through_the_reference_pool(pool, threads, whole):
    L = ckq.lib()
    T.ref_pool_set_threads(pool, threads)
    L.ckq_set_parallel_whole(whole)
    for fmt, name, M, K in (("q4_k", "gemv_q4_k_q8_k_parallel_dispatch", 4101, 4096),
                            ("q6_k", "gemv_q6_k_q8_k_parallel_dispatch", 1000, 2048),
                            ("q8_0", "gemv_q8_0_q8_0_parallel_dispatch", 3003, 896)):
        W = T.synth_weights(fmt, M, K, seed=threads + M)
        xq = T.oracle_quantize(T.normal(K, 0.0, 1.0, 9), T.act_fmt(fmt))
        y = np.full(M, 7.0, np.float32)
        say("pool dispatch", name, "threads", threads, "whole" if whole else "rows")
        for _ in range(3):                          # repeated dispatches reuse the pool's barrier
            getattr(pool, name)(T.ptr(y), T.ptr(W), T.ptr(xq), M, K)
        serial = P.gemv(fmt, W, xq, M, K)
        assert np.array_equal(y, serial), fmt
        assert T.norm_err(y, T.oracle_gemv(fmt, W, xq, M, K)) <= 1e-4, fmt


@pytest.mark.parametrize("threads", [8, 16])
def test_q5_k_dispatch_hands_each_thread_a_row_slice(pool, threads):
    """gemv_q5_k_parallel_dispatch splits the rows itself and calls gemv_q5_k on
    sub-matrices (pointers into W), with fp32 activations (ck_parallel_decode.c:150-166, 243-258)."""
    L = ckq.lib()
    T.ref_pool_set_threads(pool, threads)
    L.ckq_set_parallel_whole(0)
    M, K = 4864, 1024
    W = T.synth_weights("q5_k", M, K, seed=threads)
    x = T.normal(K, 0.0, 1.0, 10)
    y = np.full(M, 7.0, np.float32)
    say("pool dispatch gemv_q5_k_parallel_dispatch threads", threads)
    pool.gemv_q5_k_parallel_dispatch(T.ptr(y), T.ptr(W), T.ptr(x), M, K)
    xq = T.oracle_quantize(x, "q8_k")
    assert T.norm_err(y, T.oracle_gemv("q5_k", W, xq, M, K)) <= 1e-4
    serial = np.zeros(M, np.float32)
    L.gemv_q5_k(T.ptr(serial), T.ptr(W), T.ptr(x), M, K)
    assert np.array_equal(y, serial)
