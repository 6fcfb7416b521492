"""The entry point that allocates nothing (ckq_gemm_nt_noalloc_dev): same bits
as ckq_gemm_nt_dev, which takes the partial tiles of a K-split GEMM from an
allocated workspace, on two calls in a row (the second smaller, so the static
scratch still holds the first call's partials), for every format; a split that
needs more than the static scratch is rejected with a clear error."""
import ctypes
import importlib
import sys

import numpy as np
import pytest

import ckq_testlib as T

pytestmark = pytest.mark.gpu

ckq = importlib.import_module("c-kernel-engine_amd")
P = ckq.parity
FMT = ckq.api.FMT
ESCRATCH = -4


def say(*a):
    print(*a)
    sys.stdout.flush()


def noalloc(fmt, A_t, B_t, bias_t, M, N, K):
    import torch
    c = torch.full((M * N,), 5.0, dtype=torch.float32, device="cuda")
    rc = ckq.lib().ckq_gemm_nt_noalloc_dev(FMT[fmt], P._dp(A_t), P._dp(B_t), P._dp(bias_t), P._dp(c), M, N, K, N, P._stream())
    return rc, c.view(M, N)


# (M, N, K) pairs: the first call splits K over the static scratch, the second is smaller
CASES = {
    "q4_k": [(64, 1536, 11008), (40, 1024, 4096)],     # nine K splits (3.4 MiB of partials), then four
    "q6_k": [(128, 2048, 4096), (64, 512, 2048)],      # four splits: exactly the 4 MiB the scratch holds, then two
    "q5_k": [(100, 1024, 4864), (70, 896, 2048)],
    "q8_0": [(128, 1024, 4096), (33, 1024, 2048)],     # eight splits (4 MiB), then four
}


@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q5_k", "q8_0"])
def test_noalloc_entry_point_matches_allocating_one(fmt):
    import torch
    L = ckq.lib()
    assert L.ckq_init() == 0
    L.ckq_set_gemm_policy(1)                       # matrix cores for every token count above eight: the split path
    try:
        for i, (M, N, K) in enumerate(CASES[fmt]):
            W = T.synth_weights(fmt, N, K, seed=300 + i)
            A = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 310 + i), T.act_fmt(fmt), rows=M)
            bias = T.normal(N, 0.0, 0.5, seed=320 + i) if i == 0 else None
            Wd, Ad = P.to_device(W), P.to_device(A)
            bd = None if bias is None else P.to_device(bias)
            say("no-alloc entry point", fmt, M, N, K)
            rc, got = noalloc(fmt, Ad, Wd, bd, M, N, K)
            assert rc == 0, L.ckq_error_string(rc)
            want = P.dev_gemm_nt(fmt, Ad, Wd, bd, M, N, K)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy(), want.cpu().numpy()), (M, N, K)
            rows = np.unique(np.random.default_rng(i).integers(0, N, 48))
            rb = T.row_bytes(fmt, K)
            Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
            ref = T.oracle_gemm_nt(fmt, A, Wsub, None if bias is None else bias[rows], M, len(rows), K)
            assert T.norm_err(got.cpu().numpy()[:, rows], ref) <= 1e-4
        # decode-sized calls go to the streaming kernel through the same entry point
        M, N, K = 3, 500, 1024 if fmt != "q8_0" else 896
        W = T.synth_weights(fmt, N, K, seed=330)
        A = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 331), T.act_fmt(fmt), rows=M)
        rc, got = noalloc(fmt, P.to_device(A), P.to_device(W), None, M, N, K)
        assert rc == 0
        assert np.array_equal(got.cpu().numpy(), P.dev_gemm_nt(fmt, P.to_device(A), P.to_device(W), None, M, N, K).cpu().numpy())
    finally:
        L.ckq_set_gemm_policy(0)


def test_noalloc_entry_point_leaves_device_memory_untouched():
    """The free device memory the driver reports is the same before and after
    the calls (operands and output allocated beforehand, ckq_init() done): a
    K-split matrix-core GEMM and a streaming call, several times each."""
    import torch
    L = ckq.lib()
    assert L.ckq_init() == 0
    cases = [("q4_k", 64, 1536, 11008), ("q6_k", 128, 2048, 4096), ("q4_k", 3, 500, 1024)]
    bufs = []
    for i, (fmt, M, N, K) in enumerate(cases):
        W = T.synth_weights(fmt, N, K, seed=350 + i)
        A = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 360 + i), T.act_fmt(fmt), rows=M)
        bufs.append((fmt, M, N, K, P.to_device(A), P.to_device(W), torch.zeros(M * N, dtype=torch.float32, device="cuda")))
    stream = P._stream()
    torch.cuda.synchronize()
    L.ckq_set_gemm_policy(1)
    try:
        free0 = torch.cuda.mem_get_info()[0]
        for rep in range(3):
            for fmt, M, N, K, Ad, Wd, c in bufs:
                say("no-alloc call, memory check", fmt, M, N, K, rep)
                assert L.ckq_gemm_nt_noalloc_dev(FMT[fmt], P._dp(Ad), P._dp(Wd), None, P._dp(c), M, N, K, N, stream) == 0
        torch.cuda.synchronize()
        free1 = torch.cuda.mem_get_info()[0]
    finally:
        L.ckq_set_gemm_policy(0)
    assert free1 == free0, (free0, free1)
    for fmt, M, N, K, Ad, Wd, c in bufs:          # and the results are the allocating entry point's
        L.ckq_set_gemm_policy(1)
        try:
            want = P.dev_gemm_nt(fmt, Ad, Wd, None, M, N, K)
        finally:
            L.ckq_set_gemm_policy(0)
        assert np.array_equal(c.view(M, N).cpu().numpy(), want.cpu().numpy())


def test_noalloc_entry_point_rejects_what_does_not_fit():
    """Q4_K, M = 128, N = 4096, K = 11008: four K splits of 2 MiB of partial tiles
    each exceed the 4 MiB static scratch: CKQ_ESCRATCH, nothing enqueued, output
    untouched; the allocating entry point takes the same call."""
    import torch
    L = ckq.lib()
    fmt, M, N, K = "q4_k", 128, 4096, 11008
    W = T.synth_weights(fmt, N, K, seed=340)
    A = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 341), "q8_k", rows=M)
    L.ckq_set_gemm_policy(1)
    try:
        rc, got = noalloc(fmt, P.to_device(A), P.to_device(W), None, M, N, K)
    finally:
        L.ckq_set_gemm_policy(0)
    torch.cuda.synchronize()
    assert rc == ESCRATCH
    assert b"scratch" in L.ckq_error_string(rc)
    assert (got.cpu().numpy() == 5.0).all()
    L.ckq_set_gemm_policy(1)
    try:
        ok = P.dev_gemm_nt(fmt, P.to_device(A), P.to_device(W), None, M, N, K).cpu().numpy()
    finally:
        L.ckq_set_gemm_policy(0)
    rows = np.arange(0, N, 97)
    rb = T.row_bytes(fmt, K)
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    assert T.norm_err(ok[:, rows], T.oracle_gemm_nt(fmt, A, Wsub, None, M, len(rows), K)) <= 1e-4
    # bad arguments and formats without a no-alloc form
    one = ctypes.c_void_p(256)
    assert L.ckq_gemm_nt_noalloc_dev(FMT["q5_0"], one, one, None, one, 16, 64, 64, 64, None) == -3
    assert L.ckq_gemm_nt_noalloc_dev(FMT["q4_k"], one, one, None, one, 16, 64, 100, 64, None) == -2
    assert L.ckq_gemm_nt_noalloc_dev(FMT["q4_k"], None, one, None, one, 16, 64, 256, 64, None) == -1
