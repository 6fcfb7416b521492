"""GPU parity tests: the HIP path, called through the C ABI, against the CPU
oracle on the same seeded inputs and against the golden fixtures.

Bars: quantizer outputs and integer sub-block dots bit-exact; fp32 outputs
within 1e-4 of the oracle, normalised by max|y_ref| (pointwise relative error
is not meaningful here: the reference's own builds differ from each other by
1e-3 pointwise on cancelling rows while agreeing to 1e-6 of max|y|)."""
import ctypes
import importlib
import sys

import numpy as np
import pytest

import ckq_testlib as T

pytestmark = pytest.mark.gpu

ckq = importlib.import_module("c-kernel-engine_amd")
P = ckq.parity
TOL = 1e-4
FMTS = ["q4_k", "q5_k", "q6_k", "q8_0"]


def say(*a):
    print(*a)
    sys.stdout.flush()


@pytest.fixture(scope="module", autouse=True)
def _lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    L = ckq.lib()          # raises if the HIP library is not built: no fallback
    assert L.ckq_init() == 0
    yield L
    L.ckq_weights_clear()


MATRIX_CORE_TESTS = ("mfma", "split_k", "q5_0_row_and_token")


@pytest.fixture(autouse=True)
def _gemm_policy(request, _lib):
    """Tests aimed at the matrix-core GEMMs force them for every token count
    above eight (the automatic choice would send their small shapes to the
    streaming kernel); everything else runs with the automatic choice."""
    forced = any(k in request.node.name for k in MATRIX_CORE_TESTS)
    _lib.ckq_set_gemm_policy(1 if forced else 0)
    yield
    _lib.ckq_set_gemm_policy(0)


def make_case(fmt, rows, K, kind, seed, tokens=1):
    if kind == "rand":
        W = T.random_blocks(fmt, rows * (K // T.ELEMS[fmt]), seed)
    else:
        W = T.synth_weights(fmt, rows, K, seed)
    xf = T.normal(tokens * K, 0.0, 1.0, seed + 1000)
    xq = T.oracle_quantize(xf, T.act_fmt(fmt), rows=tokens)
    return W, xf, xq


# ---- quantizers: bit-exact ------------------------------------------------------

def test_quantize_q8_k_golden_host_and_device():
    import torch
    G = T.golden()
    x, want = G["q8k_in"], G["q8k_out"]
    say("quantize_row_q8_k host path, n =", len(x))
    got = P.quantize(x, "q8_k")
    assert np.array_equal(got, want)
    say("ckq_quantize_q8_k_dev")
    got = P.dev_quantize(P.to_device(x), "q8_k").cpu().numpy()
    assert np.array_equal(got, want)
    # ck_test_ wrapper
    out = np.zeros_like(want)
    ckq.lib().ck_test_quantize_q8_k(T.ptr(x), T.ptr(out), len(x))
    assert np.array_equal(out, want)


def test_quantize_q8_0_golden_host_and_device():
    G = T.golden()
    x, want = G["q80_in"], G["q80_out"]
    say("quantize_row_q8_0 host path, n =", len(x))
    assert np.array_equal(P.quantize(x, "q8_0"), want)
    assert np.array_equal(P.dev_quantize(P.to_device(x), "q8_0").cpu().numpy(), want)


@pytest.mark.parametrize("std,seed", [(1.0, 1), (0.02, 2), (37.0, 3), (1e-6, 4)])
def test_quantize_bit_exact_vs_oracle_large(std, seed):
    rows, k = 96, 4096
    x = T.normal(rows * k, 0.0, std, seed)
    # plant ties and zero blocks
    x[0:256] = 0.0
    x[256 + 5] = 9.0 * std
    x[256 + 99] = -9.0 * std
    say("quantize q8_k / q8_0 rows=%d k=%d std=%g" % (rows, k, std))
    xd = P.to_device(x)
    for fmt in ("q8_k", "q8_0"):
        want = T.oracle_quantize(x, fmt, rows=rows)
        got = P.dev_quantize(xd, fmt, rows=rows).cpu().numpy()
        assert np.array_equal(got, want), fmt


def test_quantize_batch_equals_rows_host():
    x = T.normal(7 * 768, seed=12)
    whole = P.quantize(x, "q8_k", rows=7)
    rows = np.concatenate([P.quantize(x[r * 768:(r + 1) * 768], "q8_k") for r in range(7)])
    assert np.array_equal(whole, rows)


# ---- integer sub-block dots: bit-exact -----------------------------------------

# K values chosen to hit every lane mapping of the kernel: 4..32 positions per
# row (sub-wave rows), 64, 2-4 positions per lane, and the multi-pass loop.
K_SWEEP = {"q4_k": [256, 512, 1024, 2048, 4096, 4864, 11008, 16384, 20480],
           "q5_k": [256, 1024, 4864, 11008],
           "q6_k": [256, 512, 1024, 2048, 4096, 11008, 16384, 20480],
           "q8_0": [32, 128, 512, 896, 1024, 2048, 4096, 8192, 10240]}


@pytest.mark.parametrize("fmt", FMTS)
def test_subblock_dots_bit_exact(fmt):
    rows = 37
    for K in K_SWEEP[fmt]:
        W, _, xq = make_case(fmt, rows, K, "rand", 40 + K)
        say("subblock dots", fmt, "rows", rows, "K", K)
        got = P.dev_subblock_dots(fmt, P.to_device(W), P.to_device(xq), rows, K).cpu().numpy()
        want = T.oracle_subdots(fmt, W, xq, rows, K)
        assert np.array_equal(got, want), (fmt, K)


# ---- GEMV fp32 --------------------------------------------------------------------

@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_gemv_golden_fixture(fmt, kind):
    G = T.golden()
    M, K, _ = (int(v) for v in G["shape"])
    W = G["w_%s_%s" % (fmt, kind)]
    xq = G["act_q80" if fmt == "q8_0" else "act_q8k"]
    say("gemv golden", fmt, kind)
    y = P.gemv(fmt, W, xq, M, K)
    for build in ("avx2", "avx512"):
        assert T.norm_err(y, G["y_%s_%s_%s" % (fmt, kind, build)]) <= TOL
    c = P.gemm_nt(fmt, xq, W, G["bias"], 3, M, K)
    assert T.norm_err(c, G["c_%s_%s_avx2" % (fmt, kind)]) <= TOL


@pytest.mark.parametrize("fmt", FMTS)
def test_gemv_vs_oracle_k_sweep(fmt):
    rows = 53
    for K in K_SWEEP[fmt]:
        for kind in ("rand", "enc"):
            W, _, xq = make_case(fmt, rows, K, kind, 90 + K)
            say("gemv dev", fmt, kind, "rows", rows, "K", K)
            y = P.dev_gemm_nt(fmt, P.to_device(xq), P.to_device(W), None, 1, rows, K).cpu().numpy().reshape(-1)
            ref = T.oracle_gemv(fmt, W, xq, rows, K)
            assert T.norm_err(y, ref) <= TOL, (fmt, K, kind)
            exact = T.oracle_exact(fmt, W, xq, rows, K)
            assert T.norm_err(y, exact) <= TOL


@pytest.mark.parametrize("fmt", FMTS)
def test_gemv_row_counts(fmt):
    """Row counts around the wave/block tiling, including a single row."""
    K = 1024 if fmt != "q8_0" else 896
    for rows in (1, 2, 3, 15, 16, 17, 63, 64, 65, 127, 257):
        W, _, xq = make_case(fmt, rows, K, "rand", 7 * rows)
        say("gemv rows", fmt, rows)
        y = P.gemv(fmt, W, xq, rows, K)
        assert T.norm_err(y, T.oracle_gemv(fmt, W, xq, rows, K)) <= TOL, rows


def test_stored_bsums_semantics():
    """Q4_K/Q5_K consume the activation's STORED bsums; Q6_K never reads them
    (reference unittest/test_parallel_gemv.py:66-85 feeds zeroed bsums)."""
    G = T.golden()
    M, K, _ = (int(v) for v in G["shape"])
    xz = G["act_q8k_zero_bsums"]
    for fmt in ("q4_k", "q5_k", "q6_k"):
        for kind in ("rand", "enc"):
            say("zero bsums", fmt, kind)
            y = P.gemv(fmt, G["w_%s_%s" % (fmt, kind)], xz, M, K)
            assert T.norm_err(y, G["y_%s_%s_zero_bsums" % (fmt, kind)]) <= TOL


@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q8_0"])
def test_parallel_union_equals_serial(fmt):
    """Calling the thread-split entry point for every ith reproduces the serial
    result (reference unittest/test_parallel_gemv.py:112-170)."""
    rows, K = 301, 1024
    W, _, xq = make_case(fmt, rows, K, "rand", 5)
    serial = P.gemv(fmt, W, xq, rows, K)
    # default ("rows", the reference's semantics): every call computes exactly its own range
    ckq.lib().ckq_set_parallel_whole(-1)
    for nth in (1, 3, 8, 64):
        for simd in (False, True):
            say("parallel", fmt, "nth", nth, "simd", simd)
            y = P.gemv_parallel(fmt, W, xq, rows, K, nth, simd)
            assert np.array_equal(y, serial)
    # a single ith touches only its own rows
    y = np.full(rows, -5.0, np.float32)
    ckq.lib().gemv_q4_k_q8_k_parallel(T.ptr(y), T.ptr(W), T.ptr(xq), rows, K, 1, 4) if fmt == "q4_k" else None
    if fmt == "q4_k":
        dr = (rows + 3) // 4
        assert np.all(y[:dr] == -5.0) and np.all(y[2 * dr:] == -5.0)
        assert np.array_equal(y[dr:2 * dr], serial[dr:2 * dr])
    # "whole" mode: ith 0 computes everything, the rest return; the union is still the serial result
    ckq.lib().ckq_set_parallel_whole(1)
    try:
        assert np.array_equal(P.gemv_parallel(fmt, W, xq, rows, K, 8, True), serial)
        y = np.zeros(rows, np.float32)
        fn = getattr(ckq.lib(), P._GEMV[fmt] + "_parallel_simd")
        fn(T.ptr(y), T.ptr(W), T.ptr(xq), rows, K, 0, 8)
        assert np.array_equal(y, serial)
        y = np.full(rows, -5.0, np.float32)
        fn(T.ptr(y), T.ptr(W), T.ptr(xq), rows, K, 3, 8)     # another ith: returns at once
        assert np.all(y == -5.0)
    finally:
        ckq.lib().ckq_set_parallel_whole(-1)


# ---- batched decode / small GEMM -------------------------------------------------------

@pytest.mark.parametrize("fmt", FMTS)
def test_gemm_nt_token_counts(fmt):
    N, K = 77, 1024
    bias = T.normal(N, 0.0, 0.5, seed=8)
    for M in (1, 2, 3, 4, 5, 8, 9, 17):
        W, _, xq = make_case(fmt, N, K, "enc", 300 + M, tokens=M)
        say("gemm_nt", fmt, "tokens", M)
        ref = T.oracle_gemm_nt(fmt, xq, W, bias, M, N, K)
        c = P.gemm_nt(fmt, xq, W, bias, M, N, K)
        assert T.norm_err(c, ref) <= TOL, M
        cd = P.dev_gemm_nt(fmt, P.to_device(xq), P.to_device(W), P.to_device(bias), M, N, K).cpu().numpy()
        assert np.array_equal(cd, c)       # host and device paths run the same kernel
        # each row of a batch equals the single-token GEMV of that token
        ab = T.row_bytes(T.act_fmt(fmt), K)
        y0 = P.gemv(fmt, W, xq[(M - 1) * ab:M * ab].copy(), N, K)
        assert T.norm_err(c[M - 1] - bias, y0) <= 1e-6


def test_gemm_layouts_and_wrappers():
    """gemm_* writes Y[n*M + row]; ck_test_* quantize internally; fp32 adapters."""
    rows, K, tok = 40, 1024, 3
    L = ckq.lib()
    for fmt, gemm in (("q4_k", "gemm_q4_k_q8_k"), ("q6_k", "gemm_q6_k_q8_k")):
        W, xf, xq = make_case(fmt, rows, K, "enc", 17, tokens=tok)
        say("gemm layout", fmt)
        Y = np.zeros(tok * rows, np.float32)
        getattr(L, gemm)(T.ptr(Y), T.ptr(W), T.ptr(xq), rows, tok, K)
        ref = T.oracle_gemm_nt(fmt, xq, W, None, tok, rows, K)
        assert T.norm_err(Y.reshape(tok, rows), ref) <= TOL
        out = np.zeros(tok * rows, np.float32)
        getattr(L, "ck_test_gemm_" + fmt)(T.ptr(W), T.ptr(xf), T.ptr(out), rows, K, tok)
        assert T.norm_err(out.reshape(tok, rows), ref) <= TOL
        one = np.zeros(1, np.float32)
        getattr(L, "ck_test_gemv_" + fmt)(T.ptr(W), T.ptr(xf), T.ptr(one), K)
        assert abs(one[0] - ref[0, 0]) <= TOL * np.max(np.abs(ref))
    # Q5_K fp32 adapters
    W, xf, xq = make_case("q5_k", rows, K, "enc", 19, tokens=tok)
    y = np.zeros(rows, np.float32)
    L.gemv_q5_k(T.ptr(y), T.ptr(W), T.ptr(xf), rows, K)
    assert T.norm_err(y, T.oracle_gemv("q5_k", W, xq, rows, K)) <= TOL
    bias = T.normal(rows, seed=3)
    c = np.zeros(tok * rows, np.float32)
    L.gemm_nt_q5_k(T.ptr(xf), T.ptr(W), T.ptr(bias), T.ptr(c), tok, rows, K)
    assert T.norm_err(c.reshape(tok, rows), T.oracle_gemm_nt("q5_k", xq, W, bias, tok, rows, K)) <= TOL
    # Q8_0: vec_dot, fp32-activation GEMV, ck_test wrappers
    W, xf, xq = make_case("q8_0", rows, K, "enc", 23, tokens=tok)
    s = np.zeros(1, np.float32)
    L.vec_dot_q8_0_q8_0(K, T.ptr(s), T.ptr(W), T.ptr(xq))
    ref = T.oracle_gemv("q8_0", W, xq, rows, K)
    assert abs(s[0] - ref[0]) <= TOL * np.max(np.abs(ref))
    y = np.zeros(rows, np.float32)
    L.gemv_q8_0(T.ptr(y), T.ptr(W), T.ptr(xf), rows, K)
    want = np.zeros(rows, np.float32)
    T.oracle().orc_gemv_q8_0(T.ptr(want), T.ptr(W), T.ptr(xf), rows, K)
    assert T.norm_err(y, want) <= TOL
    out = np.zeros(rows, np.float32)
    L.ck_test_gemv_q8_0(T.ptr(W), T.ptr(xf), T.ptr(out), rows, K)
    assert T.norm_err(out, ref) <= TOL
    W6, _, xq6 = make_case("q6_k", 1, K, "rand", 29)
    s = np.zeros(1, np.float32)
    L.vec_dot_q6_k_q8_k(K, T.ptr(s), T.ptr(W6), T.ptr(xq6))
    assert abs(s[0] - T.oracle_gemv("q6_k", W6, xq6, 1, K)[0]) <= TOL * abs(s[0]) + 1e-6


def test_weight_cache_follows_content():
    """Same host address, new bytes: the resident copy is refreshed."""
    rows, K = 32, 1024
    W, _, xq = make_case("q4_k", rows, K, "rand", 61)
    y1 = P.gemv("q4_k", W, xq, rows, K)
    W2, _, _ = make_case("q4_k", rows, K, "rand", 62)
    W[:] = W2
    y2 = P.gemv("q4_k", W, xq, rows, K)
    assert T.norm_err(y2, T.oracle_gemv("q4_k", W2, xq, rows, K)) <= TOL
    assert T.norm_err(y1, y2) > 1e-3


# ---- full benchmark shapes ----------------------------------------------------------------

FULL = [("q4_k", 4096, 4096), ("q4_k", 11008, 4096), ("q6_k", 32000, 4096), ("q6_k", 4096, 11008),
        ("q5_k", 4864, 1024), ("q5_k", 896, 4864), ("q8_0", 151936, 896)]


@pytest.mark.parametrize("fmt,rows,K", FULL)
def test_full_size_shapes(fmt, rows, K):
    import torch
    W = T.synth_weights(fmt, rows, K, seed=rows + K)
    xf = T.normal(K, 0.0, 1.0, seed=K)
    say("full size", fmt, rows, K)
    xd = P.to_device(xf)
    xq_d = P.dev_quantize(xd, T.act_fmt(fmt))
    xq = xq_d.cpu().numpy()
    assert np.array_equal(xq, T.oracle_quantize(xf, T.act_fmt(fmt)))
    Wd = P.to_device(W)
    y = P.dev_gemm_nt(fmt, xq_d, Wd, None, 1, rows, K).cpu().numpy().reshape(-1)
    ref = T.oracle_gemv(fmt, W, xq, rows, K)
    assert T.norm_err(y, ref) <= TOL
    # size-independent properties: determinism, and linearity in the rows
    y2 = P.dev_gemm_nt(fmt, xq_d, Wd, None, 1, rows, K).cpu().numpy().reshape(-1)
    assert np.array_equal(y, y2)
    rb = T.row_bytes(fmt, K)
    perm = np.random.default_rng(1).permutation(rows)
    Wp = np.ascontiguousarray(W.reshape(rows, rb)[perm]).reshape(-1)
    yp = P.dev_gemm_nt(fmt, xq_d, P.to_device(Wp), None, 1, rows, K).cpu().numpy().reshape(-1)
    assert np.array_equal(yp, y[perm])     # a row's result does not depend on where the row sits
    torch.cuda.synchronize()


@pytest.mark.parametrize("M", [2, 4, 8])
def test_batched_decode_small_model_shapes(M):
    """Qwen2-0.5B-like shapes, M tokens (hidden 896 zero-padded to K=1024)."""
    for fmt, rows, K in (("q5_k", 896, 1024), ("q5_k", 128, 1024), ("q5_k", 4864, 1024), ("q5_k", 896, 4864),
                         ("q8_0", 4096, 896)):
        W, _, xq = make_case(fmt, rows, K, "enc", rows + M, tokens=M)
        say("batched decode", fmt, rows, K, "M", M)
        c = P.dev_gemm_nt(fmt, P.to_device(xq), P.to_device(W), None, M, rows, K).cpu().numpy()
        assert T.norm_err(c, T.oracle_gemm_nt(fmt, xq, W, None, M, rows, K)) <= TOL

# ---- fp32 activations, no activation quantization -------------------------------------------

F32_FMTS = ["q4_k", "q6_k", "q8_0"]


@pytest.mark.parametrize("fmt", F32_FMTS)
@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_f32act_golden_fixture(fmt, kind):
    """gemv_q4_k / gemv_q6_k / gemm_nt_q4_k / _q6_k / _q8_0 through the drop-in
    symbols (host pointers) against the reference builds' own outputs."""
    G = T.golden()
    M, K, TOK = (int(v) for v in G["shape"])
    W, xf, bias = G["w_%s_%s" % (fmt, kind)], G["act_f32"], G["bias"]
    say("f32act golden", fmt, kind)
    c = P.gemm_nt_f32act(fmt, xf, W, bias, TOK, M, K)
    for build in ("avx2", "avx512"):
        assert T.norm_err(c.reshape(-1), G["c_%s_%s_f32w_%s" % (fmt, kind, build)]) <= TOL
    if fmt != "q8_0":
        y = P.gemv_f32act(fmt, W, xf, M, K)
        assert T.norm_err(y, G["y_%s_%s_f32w_avx2" % (fmt, kind)]) <= TOL
        assert ckq.lib().dot_q4_k is not None
    Y = P.gemm_f32act(fmt, W, xf, M, TOK, K)                   # Y[n*M + row]
    assert T.norm_err(Y, T.oracle_gemm_nt_f32act(fmt, xf, W, None, TOK, M, K)) <= TOL
    if fmt == "q4_k":
        import ctypes as C
        r = ckq.lib().dot_q4_k(C.c_void_p(W.ctypes.data), C.c_void_p(xf.ctypes.data), K)
        assert abs(r - y[0]) <= TOL * max(1.0, np.abs(y).max())


@pytest.mark.parametrize("fmt", F32_FMTS)
def test_f32act_vs_oracle_shapes(fmt):
    """Ragged row counts, short and long rows, several tokens, device pointers."""
    blk = 32 if fmt == "q8_0" else 256
    for rows, K, M in ((1, blk, 1), (7, 2 * blk, 3), (130, 1024, 2), (257, 4096, 1), (33, 11008 if fmt != "q8_0" else 896, 5)):
        W, xf, _ = make_case(fmt, rows, K, "rand" if rows % 2 else "enc", rows + K, tokens=M)
        bias = T.normal(rows, 0.0, 0.5, seed=rows)
        say("f32act", fmt, rows, K, "M", M)
        c = P.dev_gemm_nt_f32act(fmt, P.to_device(xf), P.to_device(W), P.to_device(bias), M, rows, K).cpu().numpy()
        assert T.norm_err(c.reshape(M, rows), T.oracle_gemm_nt_f32act(fmt, xf, W, bias, M, rows, K)) <= TOL
        # K not a multiple of the block size: nothing is written
    out = np.full(4, 7.0, np.float32)
    getattr(ckq.lib(), "gemv_" + fmt)(P._p(out), P._p(np.zeros(4096, np.uint8)), P._p(np.zeros(100, np.float32)), 4, 100)
    assert np.all(out == 7.0)


def test_f32act_full_size():
    """11008 x 4096 Q4_K with fp32 activations against dequantize-then-matmul in fp64."""
    rows, K = 11008, 4096
    W, xf, _ = make_case("q4_k", rows, K, "enc", 77)
    say("f32act full size")
    y = P.dev_gemm_nt_f32act("q4_k", P.to_device(xf), P.to_device(W), None, 1, rows, K).cpu().numpy().reshape(-1)
    want = T.np_dequant("q4_k", W).reshape(rows, K).astype(np.float64) @ xf.astype(np.float64)
    assert T.norm_err(y, want) <= TOL

# ---- fused producer: rmsnorm -> Q8_K, bit-exact -----------------------------------------------

def test_rmsnorm_q8_k_fused_golden_host_and_device():
    G = T.golden()
    TF, DF, AF = (int(v) for v in G["rms_shape"])
    x, g, eps = G["rms_in"], G["rms_gamma"], float(G["rms_eps"][0])
    say("rmsnorm_q8_k_fused golden")
    assert np.array_equal(P.rmsnorm_q8_k_fused(x, g, TF, DF, AF, eps), G["rms_out"])
    out = P.dev_rmsnorm_q8_k_fused(P.to_device(x), P.to_device(g), TF, DF, AF, eps).cpu().numpy()
    assert np.array_equal(out, G["rms_out"])


@pytest.mark.parametrize("tokens,D,std,seed", [(1, 256, 1.0, 1), (5, 4096, 1.0, 2), (64, 1024, 30.0, 3),
                                                (3, 11008 // 256 * 256, 1e-3, 4), (512, 4096, 2.0, 5)])
def test_rmsnorm_q8_k_fused_bit_exact_vs_oracle(tokens, D, std, seed):
    x = T.normal(tokens * D, 0.0, std, seed)
    g = T.normal(D, 1.0, 0.3, seed + 50)
    say("rmsnorm_q8_k_fused", tokens, D, std)
    ref = np.zeros(tokens * (D // 256) * 292, np.uint8)
    T.oracle().orc_rmsnorm_q8_k_fused(T.ptr(x), T.ptr(g), T.ptr(ref), tokens, D, D, ctypes.c_float(1e-6))
    out = P.dev_rmsnorm_q8_k_fused(P.to_device(x), P.to_device(g), tokens, D).cpu().numpy()
    assert np.array_equal(out, ref)
    if tokens <= 8:
        # feeding the GEMV: same result as quantized-activation GEMV on the oracle's blocks
        W = T.synth_weights("q4_k", 64, D, seed + 9)
        y = P.dev_gemm_nt("q4_k", P.to_device(out), P.to_device(W), None, tokens, 64, D).cpu().numpy()
        assert T.norm_err(y, T.oracle_gemm_nt("q4_k", ref, W, None, tokens, 64, D)) <= TOL

# ---- row dequantizers and quantized embedding lookup, bit-exact -----------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q8_0"])
def test_dequant_rows_bit_exact(fmt):
    G = T.golden()
    w, want = G["deq_%s_w" % fmt], G["deq_%s_out" % fmt]
    say("dequant row golden", fmt)
    assert np.array_equal(P.dequant_row(fmt, w, len(want)).view(np.uint32), want.view(np.uint32))
    if fmt != "q8_0":
        # the parity scripts' name for the same routine (reference src/ck_parity_api.c:189-197)
        out = np.zeros(len(want), np.float32)
        getattr(ckq.lib(), "ck_test_dequant_" + fmt)(T.ptr(w), T.ptr(out), len(want))
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    # larger, against the oracle
    n = 64 * 1024
    W = T.random_blocks(fmt, n // T.ELEMS[fmt], 91)
    ref = np.zeros(n, np.float32)
    getattr(T.oracle(), "orc_dequant_%s_row" % fmt)(T.ptr(W), T.ptr(ref), ctypes.c_size_t(n))
    got = P.dev_dequant_rows(fmt, P.to_device(W), None, 0, None, n, n, 1, 1).cpu().numpy().reshape(-1)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("add_pos", [0, 1])
def test_embedding_forward_golden_and_oracle(fmt, add_pos):
    G = T.golden()
    VOC, ED, AED, CTX, NTOK = (int(v) for v in G["emb_shape"])
    ids, pos, tab = G["emb_ids"], G["emb_pos"], G["emb_table_" + fmt]
    say("embedding golden", fmt, add_pos)
    out = P.embedding_forward(fmt, ids, NTOK, VOC, tab, pos, ED, AED, CTX, add_pos, fill=9.0)
    assert np.array_equal(out.reshape(-1).view(np.uint32), G["emb_out_%s_pos%d" % (fmt, add_pos)].view(np.uint32))
    # a model-sized lookup on the device: 64 tokens of a 32000 x 4096 table (Q8_0: 151936 x 896)
    voc, dim = (151936, 896) if fmt == "q8_0" else (32000, 4096)
    tabL = T.random_blocks(fmt, voc * (dim // T.ELEMS[fmt]), 92)
    idsL = np.random.default_rng(5).integers(-3, voc + 3, size=64).astype(np.int32)
    posL = T.normal(80 * dim, 0.0, 0.1, seed=93)
    ref = np.full(80 * dim, 9.0, np.float32)
    T.oracle().orc_embedding_forward(T.FMT[fmt], T.ptr(idsL), 64, voc, T.ptr(tabL), T.ptr(posL), T.ptr(ref), dim - 8, dim, 80, add_pos)
    got = P.dev_dequant_rows(fmt, P.to_device(tabL), P.to_device(idsL), voc, P.to_device(posL) if add_pos else None,
                             dim - 8, dim, 64, 80).cpu().numpy().reshape(-1)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


# ---- prefill GEMM on the matrix cores (Q4_K, token counts above 16) -------------------------

@pytest.mark.parametrize("M,N,K", [(17, 128, 256), (33, 200, 1024), (64, 96, 512), (100, 333, 2048),
                                   (128, 1, 256), (65, 129, 4096)])
def test_gemm_mfma_q4_k_vs_oracle(M, N, K):
    bias = T.normal(N, 0.0, 0.5, seed=N)
    for kind in ("rand", "enc"):
        W, _, xq = make_case("q4_k", N, K, kind, 700 + M + N, tokens=M)
        say("gemm mfma q4_k", kind, "M", M, "N", N, "K", K)
        ref = T.oracle_gemm_nt("q4_k", xq, W, bias, M, N, K)
        c = P.dev_gemm_nt("q4_k", P.to_device(xq), P.to_device(W), P.to_device(bias), M, N, K).cpu().numpy()
        assert T.norm_err(c, ref) <= TOL, (M, N, K, kind)
        # the matrix-core path and the dot4 path agree token by token
        ab = T.row_bytes("q8_k", K)
        y = P.gemv("q4_k", W, xq[(M - 1) * ab:M * ab].copy(), N, K)
        assert T.norm_err(c[M - 1] - bias, y) <= 2e-6
        ch = P.gemm_nt("q4_k", xq, W, bias, M, N, K)      # host-pointer entry point, same kernel
        assert np.array_equal(ch, c)


def test_gemm_mfma_stored_bsums_and_extremes():
    """Stored bsums are consumed (zeroed bsums drop the min term), and the
    extreme quant values (nibble 15, scale 63, q8 = -128/127) stay exact."""
    M, N, K = 64, 64, 512
    W, _, xq = make_case("q4_k", N, K, "rand", 911, tokens=M)
    xz = xq.copy().reshape(-1, 292)
    xz[:, 260:292] = 0
    xz = xz.reshape(-1)
    ref = T.oracle_gemm_nt("q4_k", xz, W, None, M, N, K)
    c = P.dev_gemm_nt("q4_k", P.to_device(xz), P.to_device(W), None, M, N, K).cpu().numpy()
    assert T.norm_err(c, ref) <= TOL
    # extremes: all nibbles 15, all scales/mins 63, activations alternating -128 / 127
    Wb = W.copy().reshape(-1, 144)
    Wb[:, 4:16] = 0xFF
    Wb[:, 16:] = 0xFF
    Wb = Wb.reshape(-1)
    xb = xq.copy().reshape(-1, 292)
    q = np.where(np.arange(256) % 2 == 0, -128, 127).astype(np.int8)
    xb[:, 4:260] = q.view(np.uint8)
    xb[:, 260:292] = np.tile(np.array([-8] * 16, np.int16).view(np.uint8), 1)
    xb = xb.reshape(-1)
    ref = T.oracle_gemm_nt("q4_k", xb, Wb, None, M, N, K)
    c = P.dev_gemm_nt("q4_k", P.to_device(xb), P.to_device(Wb), None, M, N, K).cpu().numpy()
    assert T.norm_err(c, ref) <= TOL
    # largest positive dot: activations all 127
    xb = xb.reshape(-1, 292)
    xb[:, 4:260] = 127
    xb[:, 260:292] = np.array([127 * 16] * 16, np.int16).view(np.uint8)
    xb = xb.reshape(-1)
    ref = T.oracle_gemm_nt("q4_k", xb, Wb, None, M, N, K)
    c = P.dev_gemm_nt("q4_k", P.to_device(xb), P.to_device(Wb), None, M, N, K).cpu().numpy()
    assert T.norm_err(c, ref) <= TOL


def test_gemm_mfma_full_prefill_shape():
    """M=512, N=11008, K=4096.  The oracle is evaluated on a sample of weight
    rows (the whole product would take minutes on the CPU); every token is
    checked for those rows, and the GEMM is checked against the GEMV kernel on
    whole rows of C for a few tokens."""
    M, N, K = 512, 11008, 4096
    W = T.synth_weights("q4_k", N, K, seed=5150)
    xf = T.normal(M * K, 0.0, 1.0, seed=5151)
    bias = T.normal(N, 0.0, 0.5, seed=5152)
    say("gemm mfma full prefill shape")
    xq_d = P.dev_quantize(P.to_device(xf), "q8_k", rows=M)
    xq = xq_d.cpu().numpy()
    Wd, bd = P.to_device(W), P.to_device(bias)
    c = P.dev_gemm_nt("q4_k", xq_d, Wd, bd, M, N, K).cpu().numpy()
    rb = T.row_bytes("q4_k", K)
    rows = np.array([0, 1, 31, 32, 127, 128, 5000, 5503, 5504, 8191, 8192, 9000, 11006, 11007])
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    ref = T.oracle_gemm_nt("q4_k", xq, Wsub, np.ascontiguousarray(bias[rows]), M, len(rows), K)
    assert T.norm_err(c[:, rows], ref) <= TOL
    ab = T.row_bytes("q8_k", K)
    for t in (0, 63, 64, 300, 511):
        y = P.dev_gemm_nt("q4_k", P.to_device(xq[t * ab:(t + 1) * ab].copy()), Wd, bd, 1, N, K).cpu().numpy().reshape(-1)
        assert T.norm_err(c[t], y) <= 2e-6, t
    assert np.array_equal(P.dev_gemm_nt("q4_k", xq_d, Wd, bd, M, N, K).cpu().numpy(), c)


@pytest.mark.parametrize("fmt", ["q4_k", "q6_k"])
def test_gemm_mfma_more_tiles_than_block_slots(fmt):
    """A ragged grid larger than the chip holds at once (549 tiles of 64 tokens
    x 128 rows for Q4_K, nine K-blocks), with a bias: blocks of a second round
    start while others still run.  Oracle on weight rows spread over the row
    tiles for every token, whole rows against the GEMV kernel for a few tokens,
    same bits on a second run."""
    M, N, K = 520, 7700, 2304
    W = T.synth_weights(fmt, N, K, seed=5350)
    xf = T.normal(M * K, 0.0, 1.0, seed=5351)
    bias = T.normal(N, 0.0, 0.5, seed=5352)
    say("gemm mfma more tiles than slots", fmt)
    af = P.act_format(fmt)
    xq_d = P.dev_quantize(P.to_device(xf), af, rows=M)
    xq = xq_d.cpu().numpy()
    Wd, bd = P.to_device(W), P.to_device(bias)
    c = P.dev_gemm_nt(fmt, xq_d, Wd, bd, M, N, K).cpu().numpy()
    rb = T.row_bytes(fmt, K)
    rows = np.array([0, 127, 128, 3583, 3584, 7039, 7040, 7167, 7168, 7169, 7423, 7424, 7679, 7680, 7698, 7699])
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    ref = T.oracle_gemm_nt(fmt, xq, Wsub, np.ascontiguousarray(bias[rows]), M, len(rows), K)
    assert T.norm_err(c[:, rows], ref) <= TOL
    ab = T.row_bytes(af, K)
    for t in (0, 63, 64, 300, 511, 512, 519):
        y = P.dev_gemm_nt(fmt, P.to_device(xq[t * ab:(t + 1) * ab].copy()), Wd, bd, 1, N, K).cpu().numpy().reshape(-1)
        assert T.norm_err(c[t], y) <= 2e-6, t
    assert np.array_equal(P.dev_gemm_nt(fmt, xq_d, Wd, bd, M, N, K).cpu().numpy(), c)


# ---- prefill GEMM on the matrix cores, Q6_K (token counts above 16) --------------------------

@pytest.mark.parametrize("M,N,K", [(17, 128, 256), (33, 200, 1024), (64, 96, 512), (100, 333, 2048),
                                   (128, 1, 256), (65, 129, 4096),
                                   (130, 8320, 256), (512, 4224, 512)])    # the last two use 128-token tiles
def test_gemm_mfma_q6_k_vs_oracle(M, N, K):
    bias = T.normal(N, 0.0, 0.5, seed=N)
    for kind in ("rand", "enc"):
        W, _, xq = make_case("q6_k", N, K, kind, 900 + M + N, tokens=M)
        say("gemm mfma q6_k", kind, "M", M, "N", N, "K", K)
        ref = T.oracle_gemm_nt("q6_k", xq, W, bias, M, N, K)
        c = P.dev_gemm_nt("q6_k", P.to_device(xq), P.to_device(W), P.to_device(bias), M, N, K).cpu().numpy()
        assert T.norm_err(c, ref) <= TOL, (M, N, K, kind)
        # the matrix-core path and the dot4 path agree token by token
        ab = T.row_bytes("q8_k", K)
        for t in (0, M - 1):
            y = P.gemv("q6_k", W, xq[t * ab:(t + 1) * ab].copy(), N, K)
            assert T.norm_err(c[t], y + bias) <= 2e-6
        if N <= 512:
            ch = P.gemm_nt("q6_k", xq, W, bias, M, N, K)      # host-pointer entry point, same kernel
            assert np.array_equal(ch, c)


def test_gemm_mfma_q6_k_extremes():
    """The scaled weight sc * (q - 32) spans [-4064, 4096]; the corners of that
    range and the extreme activations stay exact through the two int8 planes."""
    M, N, K = 64, 64, 512
    W, _, xq = make_case("q6_k", N, K, "rand", 977, tokens=M)
    for ql, qh, sc in ((0x00, 0x00, -128), (0xFF, 0xFF, 127), (0x00, 0x00, 127), (0xFF, 0xFF, -128)):
        Wb = W.copy().reshape(-1, 210)
        Wb[:, 0:128] = ql
        Wb[:, 128:192] = qh
        Wb[:, 192:208] = np.uint8(sc & 0xFF)
        Wb = Wb.reshape(-1)
        for pattern in ("alt", "max", "min"):
            xb = xq.copy().reshape(-1, 292)
            q = {"alt": np.where(np.arange(256) % 2 == 0, -128, 127), "max": np.full(256, 127),
                 "min": np.full(256, -128)}[pattern].astype(np.int8)
            xb[:, 4:260] = q.view(np.uint8)
            xb[:, 260:292] = q.astype(np.int16).reshape(16, 16).sum(axis=1).astype(np.int16).view(np.uint8)
            xb = xb.reshape(-1)
            say("gemm mfma q6_k extremes", ql, sc, pattern)
            ref = T.oracle_gemm_nt("q6_k", xb, Wb, None, M, N, K)
            c = P.dev_gemm_nt("q6_k", P.to_device(xb), P.to_device(Wb), None, M, N, K).cpu().numpy()
            assert T.norm_err(c, ref) <= TOL, (ql, sc, pattern)


def test_gemm_mfma_q6_k_down_projection_shape():
    """M=512, N=4096, K=11008: the oracle on a sample of weight rows for every
    token, and whole rows of C against the GEMV kernel for a few tokens."""
    M, N, K = 512, 4096, 11008
    W = T.synth_weights("q6_k", N, K, seed=6160)
    xf = T.normal(M * K, 0.0, 1.0, seed=6161)
    say("gemm mfma q6_k down projection shape")
    xq_d = P.dev_quantize(P.to_device(xf), "q8_k", rows=M)
    xq = xq_d.cpu().numpy()
    Wd = P.to_device(W)
    c = P.dev_gemm_nt("q6_k", xq_d, Wd, None, M, N, K).cpu().numpy()
    rb = T.row_bytes("q6_k", K)
    rows = np.array([0, 1, 31, 32, 127, 128, 2047, 2048, 4094, 4095])
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    ref = T.oracle_gemm_nt("q6_k", xq, Wsub, None, M, len(rows), K)
    assert T.norm_err(c[:, rows], ref) <= TOL
    ab = T.row_bytes("q8_k", K)
    for t in (0, 63, 64, 300, 511):
        y = P.dev_gemm_nt("q6_k", P.to_device(xq[t * ab:(t + 1) * ab].copy()), Wd, None, 1, N, K).cpu().numpy().reshape(-1)
        assert T.norm_err(c[t], y) <= 2e-6, t


# ---- fused prefill MLP ------------------------------------------------------------------------

def _q8k_fields(b):
    b = b.reshape(-1, 292)
    return b[:, :4].copy().view(np.float32).reshape(-1), b[:, 4:260].view(np.int8).astype(np.int32), \
        b[:, 260:].copy().view(np.int16).astype(np.int32)


def test_swiglu_q8_k_vs_oracle():
    """SiLU(gate)*up quantized to Q8_K.  The device rounds exp once from double,
    the host's expf is almost always correctly rounded too: block scales agree to
    one unit in the last place, quants differ by at most one in a vanishing
    fraction, and the stored bsums are the sums of the stored quants."""
    rows, k, ld = 37, 1024, 2 * 1024 + 64
    g = T.normal(rows * ld, 0.0, 3.0, seed=4401)
    u = T.normal(rows * ld, 0.0, 1.0, seed=4402)
    g.reshape(rows, ld)[3, 256:512] = 0.0                   # SiLU(0) = 0: a zero block
    g.reshape(rows, ld)[5, :k] *= 30.0                      # saturated SiLU on both sides
    want = np.zeros(rows * (k // 256) * 292, np.uint8)
    T.oracle().orc_swiglu_q8_k(T.ptr(g), T.ptr(u), T.ptr(want), rows, k, ld)
    say("ckq_swiglu_q8_k_dev rows", rows, "k", k, "ld", ld)
    got = P.dev_swiglu_q8_k(P.to_device(g), P.to_device(u), rows, k, ld).cpu().numpy()
    dg, qg, bg = _q8k_fields(got)
    dw, qw, bw = _q8k_fields(want)
    assert np.all(np.abs(dg - dw) <= 1.2e-7 * np.abs(dw))
    assert np.abs(qg - qw).max() <= 1 and np.count_nonzero(qg != qw) <= qg.size // 5000
    assert np.array_equal(bg, qg.reshape(-1, 16, 16).sum(axis=2))
    assert not got.reshape(-1, 292)[3 * (k // 256) + 1].any()


@pytest.mark.parametrize("fmt", ["q4_k", "q6_k"])
def test_fused_mlp_golden_case(fmt):
    """The reference's own output for 70 tokens (host pointers, then device pointers)."""
    G = T.golden()
    SEQ, ED, AED, ID, AID = (int(v) for v in G["mlp_shape"])
    x, w1, b1, b2, w2 = G["mlp_x"], G["mlp_w1"], G["mlp_b1"], G["mlp_b2"], G["mlp_w2_" + fmt]
    want = G["mlp_out_%s_avx2" % fmt].reshape(SEQ, AED)
    say("fused_mlp_swiglu_prefill_w1w2_quant golden", fmt)
    got = P.fused_mlp_swiglu_prefill_w1w2_quant(x, w1, b1, "q8_0", w2, b2, fmt, SEQ, ED, AED, ID, AID)
    assert T.norm_err(got, want) <= TOL
    import torch
    out_d = torch.zeros(SEQ * AED, dtype=torch.float32, device="cuda")
    scr = torch.zeros(16, dtype=torch.uint8, device="cuda")
    d = [P.to_device(a) for a in (x, w1, b1, w2, b2)]          # kept alive across the call
    ckq.lib().fused_mlp_swiglu_prefill_w1w2_quant(
        P._dp(d[0]), P._dp(d[1]), P._dp(d[2]), P.CK_DT["q8_0"], P._dp(d[3]), P._dp(d[4]), P.CK_DT[fmt], P._dp(out_d),
        SEQ, ED, AED, ID, AID, P._dp(scr))
    assert np.array_equal(out_d.cpu().numpy().reshape(SEQ, AED), got)


@pytest.mark.parametrize("fmt,seq,E,I,bias", [("q4_k", 130, 896, 4864, True), ("q6_k", 33, 256, 1024, False),
                                              ("q4_k", 1, 64, 256, True), ("q6_k", 512, 128, 512, True)])
def test_fused_mlp_vs_oracle(fmt, seq, E, I, bias):
    """Stage by stage, each stage of the oracle fed with the device's previous
    stage: between the two GEMMs sits a quantizer, and a last-place difference
    in a gate value (the GEMMs sum in different orders) can move one quant by a
    whole step, which no fp32 tolerance on the end result accounts for.  The
    fused call must equal the chain of its stages bit for bit, and stay within
    a few quantization flips of the all-CPU result end to end."""
    import torch
    x = T.normal(seq * E, 0.0, 1.0, seed=4500 + seq)
    w1 = T.synth_weights("q8_0", 2 * I, E, seed=4501 + seq, std=0.25)
    w2 = T.synth_weights(fmt, E, I, seed=4502 + seq)
    b1 = T.normal(2 * I, 0.0, 0.3, seed=4503) if bias else None
    b2 = T.normal(E, 0.0, 0.3, seed=4504) if bias else None
    say("fused mlp", fmt, "seq", seq, "E", E, "I", I, "bias", bias)
    got = P.fused_mlp_swiglu_prefill_w1w2_quant(x, w1, b1, "q8_0", w2, b2, fmt, seq, E, E, I, I)
    # stage 1: Q8_0 of x, bit-exact
    xq_d = P.dev_quantize(P.to_device(x), "q8_0", rows=seq)
    xq = xq_d.cpu().numpy()
    assert np.array_equal(xq, T.oracle_quantize(x, "q8_0", rows=seq))
    # stage 2: gate and up in one GEMM over the stacked rows
    w1_d, b1_d = P.to_device(w1), (P.to_device(b1) if bias else None)
    gu_d = P.dev_gemm_nt("q8_0", xq_d, w1_d, b1_d, seq, 2 * I, E)
    gu = gu_d.cpu().numpy().reshape(seq, 2 * I)
    assert T.norm_err(gu, T.oracle_gemm_nt("q8_0", xq, w1, b1, seq, 2 * I, E)) <= TOL
    # stage 3: SiLU(gate)*up -> Q8_K, oracle applied to the device's gate and up
    h_d = P.dev_swiglu_q8_k(gu_d, gu_d.view(-1)[I:], seq, I, 2 * I)
    h = h_d.cpu().numpy()
    want_h = np.zeros_like(h)
    guc = np.ascontiguousarray(gu).reshape(-1)
    T.oracle().orc_swiglu_q8_k(T.ptr(guc), T.ptr(guc[I:]), T.ptr(want_h), seq, I, 2 * I)
    dg, qg, _ = _q8k_fields(h)
    dw, qw, _ = _q8k_fields(want_h)
    assert np.all(np.abs(dg - dw) <= 1.2e-7 * np.abs(dw))
    assert np.abs(qg - qw).max() <= 1 and np.count_nonzero(qg != qw) <= max(2, qg.size // 5000)
    # stage 4: the down GEMM on the device's Q8_K
    w2_d, b2_d = P.to_device(w2), (P.to_device(b2) if bias else None)
    out_d = P.dev_gemm_nt(fmt, h_d, w2_d, b2_d, seq, E, I)
    out = out_d.cpu().numpy().reshape(seq, E)
    assert T.norm_err(out, T.oracle_gemm_nt(fmt, h, w2, b2, seq, E, I)) <= TOL
    # the fused entry point is exactly that chain
    assert np.array_equal(got, out)
    # end to end against the all-CPU chain: fp32 tolerance plus a few quantization flips
    want = T.oracle_fused_mlp(x, w1, b1, w2, b2, fmt, seq, E, E, I, I)
    assert T.norm_err(got, want) <= 5e-3
    assert np.mean(np.abs(got - want) <= TOL * np.abs(want).max()) >= 0.98


def test_fused_mlp_argument_errors_leave_output_untouched():
    G = T.golden()
    SEQ, ED, AED, ID, AID = (int(v) for v in G["mlp_shape"])
    x, w1, w2 = G["mlp_x"], G["mlp_w1"], G["mlp_w2_q4_k"]
    mk = lambda: np.full(SEQ * AED, 7.0, np.float32)
    say("fused mlp argument errors")
    for kw in (dict(w1_fmt="q4_k"), dict(w2_fmt="q8_0")):
        out = mk()
        P.fused_mlp_swiglu_prefill_w1w2_quant(x, w1, None, kw.get("w1_fmt", "q8_0"), w2, None, kw.get("w2_fmt", "q4_k"),
                                              SEQ, ED, AED, ID, AID, output=out)
        assert np.all(out == 7.0), kw
    for dims in ((0, ED, AED, ID, AID), (SEQ, ED, AED + 8, ID, AID), (SEQ, ED, AED, ID, AID + 32),
                 (SEQ, AED + 1, AED, ID, AID), (SEQ, ED, AED, AID + 1, AID)):
        out = mk()
        P.fused_mlp_swiglu_prefill_w1w2_quant(x, w1, None, "q8_0", w2, None, "q4_k", *dims, output=out)
        assert np.all(out == 7.0), dims
    out = mk()
    P.fused_mlp_swiglu_prefill_w1w2_quant(x, w1, None, "q8_0", w2, None, "q4_k", SEQ, ED, AED, ID, AID, output=out,
                                          scratch=False)
    assert np.all(out == 7.0)
    assert int(ckq.lib().fused_mlp_swiglu_prefill_w1w2_quant_scratch_size(AED, AID)) == int(G["mlp_scratch_size"][0])


# ---- prefill GEMM on the matrix cores, Q8_0 (token counts above 16) --------------------------

@pytest.mark.parametrize("M,N,K", [(17, 128, 128), (33, 200, 96), (64, 96, 160), (100, 333, 896), (128, 1, 32),
                                   (65, 129, 4096), (130, 1030, 64), (512, 512, 416)])
def test_gemm_mfma_q8_0_vs_oracle(M, N, K):
    bias = T.normal(N, 0.0, 0.5, seed=N)
    for kind in ("rand", "enc"):
        W, _, xq = make_case("q8_0", N, K, kind, 1100 + M + N, tokens=M)
        say("gemm mfma q8_0", kind, "M", M, "N", N, "K", K)
        ref = T.oracle_gemm_nt("q8_0", xq, W, bias, M, N, K)
        c = P.dev_gemm_nt("q8_0", P.to_device(xq), P.to_device(W), P.to_device(bias), M, N, K).cpu().numpy()
        assert T.norm_err(c, ref) <= TOL, (M, N, K, kind)
        # the matrix-core path and the dot4 path agree token by token
        ab = T.row_bytes("q8_0", K)
        for t in (0, M - 1):
            y = P.gemv("q8_0", W, xq[t * ab:(t + 1) * ab].copy(), N, K)
            assert T.norm_err(c[t], y + bias) <= 2e-6
        if N <= 512:
            ch = P.gemm_nt("q8_0", xq, W, None, M, N, K)      # host-pointer entry point, same kernel, no bias
            assert T.norm_err(ch, ref - bias) <= TOL
            ldc = N + 3                                        # unaligned row pitch: scalar stores
            cd = P.to_device(np.full(M * ldc, 5.0, np.float32))
            xq_d, W_d = P.to_device(xq), P.to_device(W)        # kept alive across the call
            P.check(ckq.lib().ckq_gemm_nt_dev(P.FMT["q8_0"], P._dp(xq_d), P._dp(W_d), None, P._dp(cd),
                                              M, N, K, ldc, P._stream()), "ckq_gemm_nt_dev")
            cdn = cd.cpu().numpy().reshape(M, ldc)
            assert np.array_equal(cdn[:, :N], ch) and np.all(cdn[:, N:] == 5.0)


def test_gemm_mfma_q8_0_extremes():
    """All quants at -128 / 127 on both sides and the largest finite fp16 scales
    that keep the result finite: the int32 block sums are exact."""
    M, N, K = 64, 64, 256
    W, _, xq = make_case("q8_0", N, K, "rand", 1177, tokens=M)
    for wq, xqv in ((127, 127), (-128, -128), (-128, 127)):
        Wb = W.copy().reshape(-1, 34)
        Wb[:, 2:] = np.uint8(wq & 0xFF)
        Wb[:, 0:2] = np.array([1.5], np.float16).view(np.uint8)
        xb = xq.copy().reshape(-1, 34)
        xb[:, 2:] = np.uint8(xqv & 0xFF)
        xb[:, 0:2] = np.array([0.75], np.float16).view(np.uint8)
        say("gemm mfma q8_0 extremes", wq, xqv)
        ref = T.oracle_gemm_nt("q8_0", xb.reshape(-1), Wb.reshape(-1), None, M, N, K)
        c = P.dev_gemm_nt("q8_0", P.to_device(xb.reshape(-1)), P.to_device(Wb.reshape(-1)), None, M, N, K).cpu().numpy()
        assert np.array_equal(c, ref)        # every term is exact in fp32 here
        assert c[0, 0] == np.float32(1.5 * 0.75 * wq * xqv * 32 * (K // 32))


# ---- prefill GEMM on the matrix cores, Q5_K (token counts above 16) --------------------------

@pytest.mark.parametrize("M,N,K", [(65, 128, 256), (70, 200, 1024), (66, 96, 512), (100, 333, 2048),
                                   (128, 1, 256), (97, 129, 4864), (512, 896, 1024)])
def test_gemm_mfma_q5_k_vs_oracle(M, N, K):
    bias = T.normal(N, 0.0, 0.5, seed=N)
    for kind in ("rand", "enc"):
        W, _, xq = make_case("q5_k", N, K, kind, 1300 + M + N, tokens=M)
        say("gemm mfma q5_k", kind, "M", M, "N", N, "K", K)
        ref = T.oracle_gemm_nt("q5_k", xq, W, bias, M, N, K)
        c = P.dev_gemm_nt("q5_k", P.to_device(xq), P.to_device(W), P.to_device(bias), M, N, K).cpu().numpy()
        assert T.norm_err(c, ref) <= TOL, (M, N, K, kind)
        # the matrix-core path and the dot4 path agree token by token
        ab = T.row_bytes("q8_k", K)
        for t in (0, M - 1):
            y = P.gemv("q5_k", W, xq[t * ab:(t + 1) * ab].copy(), N, K)
            assert T.norm_err(c[t], y + bias) <= 2e-6
        if N <= 512:
            ch = P.gemm_nt("q5_k", xq, W, bias, M, N, K)      # host-pointer entry point, same kernel
            assert np.array_equal(ch, c)


def test_gemm_mfma_q5_k_stored_bsums_and_extremes():
    """Stored bsums are consumed (zeroed bsums drop the min term), and the
    extreme values (5-bit value 31, scale and min 63, q8 = -128 / 127, bsums at
    both ends of their range) stay exact through the byte-split operands."""
    M, N, K = 96, 64, 512
    W, _, xq = make_case("q5_k", N, K, "rand", 1311, tokens=M)
    xz = xq.copy().reshape(-1, 292)
    xz[:, 260:292] = 0
    xz = xz.reshape(-1)
    say("gemm mfma q5_k zeroed bsums")
    ref = T.oracle_gemm_nt("q5_k", xz, W, None, M, N, K)
    c = P.dev_gemm_nt("q5_k", P.to_device(xz), P.to_device(W), None, M, N, K).cpu().numpy()
    assert T.norm_err(c, ref) <= TOL
    Wb = W.copy().reshape(-1, 176)
    Wb[:, 4:16] = 0xFF          # all scales and mins 63
    Wb[:, 16:] = 0xFF           # all fifth bits and nibbles set: every value 31
    Wb = Wb.reshape(-1)
    for pattern in ("alt", "max", "min"):
        xb = xq.copy().reshape(-1, 292)
        q = {"alt": np.where(np.arange(256) % 2 == 0, -128, 127), "max": np.full(256, 127),
             "min": np.full(256, -128)}[pattern].astype(np.int8)
        xb[:, 4:260] = q.view(np.uint8)
        xb[:, 260:292] = q.astype(np.int16).reshape(16, 16).sum(axis=1).astype(np.int16).view(np.uint8)
        xb = xb.reshape(-1)
        say("gemm mfma q5_k extremes", pattern)
        ref = T.oracle_gemm_nt("q5_k", xb, Wb, None, M, N, K)
        c = P.dev_gemm_nt("q5_k", P.to_device(xb), P.to_device(Wb), None, M, N, K).cpu().numpy()
        assert T.norm_err(c, ref) <= TOL, pattern


# ---- loader hook: registered weight regions ---------------------------------------------------

def test_weights_register_manifest_and_ranges(tmp_path):
    """A weight arena laid out by a manifest (as the reference's loader fills it):
    the hook uploads the quantized tensors once; calls with host pointers into
    the arena - whole tensors, row ranges of them, the gate or up half of a
    stacked matrix - are served from those regions without new uploads."""
    L = ckq.lib()
    L.ckq_weights_clear()
    N, K = 48, 512
    wa = T.synth_weights("q4_k", N, K, seed=9101)
    wb = T.synth_weights("q6_k", N, K, seed=9102)
    arena = np.zeros(4096 + len(wa) + 64 + len(wb) + 512, np.uint8)
    oa, ob = 4096, 4096 + len(wa) + 64
    arena[oa:oa + len(wa)] = wa
    arena[ob:ob + len(wb)] = wb
    arena[:4096].view(np.float32)[:] = 1.0                       # an fp32 tensor the hook must skip
    m = tmp_path / "weights_manifest.map"
    m.write_text("# name|dtype|file_offset|size|runtime_offset\n"
                 "model.norm.weight|fp32|8|4096|0\n"
                 "model.layers.0.wq|Q4_K|4104|%d|%d\n"
                 "model.layers.0.wdown|q6k|0x%x|%d|%d\n" % (len(wa), oa, 4104 + len(wa), len(wb), ob))
    say("ckq_weights_register_manifest")
    assert L.ckq_weights_register_manifest(T.ptr(arena), str(m).encode()) == 2
    nbytes = ctypes.c_size_t(0)
    assert L.ckq_weights_resident(ctypes.byref(nbytes)) == 2 and nbytes.value == len(wa) + len(wb)
    xq = T.oracle_quantize(T.normal(K, seed=9103), "q8_k")
    ya = P.gemv("q4_k", arena[oa:oa + len(wa)], xq, N, K)          # views: host pointers into the arena
    yb = P.gemv("q6_k", arena[ob:ob + len(wb)], xq, N, K)
    assert T.norm_err(ya, T.oracle_gemv("q4_k", wa, xq, N, K)) <= TOL
    assert T.norm_err(yb, T.oracle_gemv("q6_k", wb, xq, N, K)) <= TOL
    rb = T.row_bytes("q4_k", K)
    ysub = P.gemv("q4_k", arena[oa + 8 * rb:oa + 40 * rb], xq, 32, K)   # rows 8..39 of the first tensor
    assert np.array_equal(ysub, ya[8:40])
    assert L.ckq_weights_resident(None) == 2                       # nothing new was uploaded
    # a registered region is not re-checked: new content needs invalidate
    arena[oa:oa + len(wa)] = T.synth_weights("q4_k", N, K, seed=9104)
    assert np.array_equal(P.gemv("q4_k", arena[oa:oa + len(wa)], xq, N, K), ya)
    L.ckq_weights_invalidate(T.ptr(arena[oa:]))
    assert L.ckq_weights_resident(None) == 1
    y2 = P.gemv("q4_k", arena[oa:oa + len(wa)], xq, N, K)
    assert T.norm_err(y2, T.oracle_gemv("q4_k", arena[oa:oa + len(wa)].copy(), xq, N, K)) <= TOL
    L.ckq_weights_clear()
    assert L.ckq_weights_resident(None) == 0


# ---- K-split prefill GEMMs ----------------------------------------------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
def test_gemm_split_k_is_deterministic_and_matches_oracle(fmt):
    """Few tiles and a long K: the launch splits K over several blocks per tile
    and sums the partial tiles in a fixed order.  Same bits on every run, the
    oracle's values within the fp32 tolerance, bias added once."""
    M, N, K = 96, 200, 19 * 256          # 4 tiles, 19 (or 38) K-steps: a ragged last split
    bias = T.normal(N, 0.0, 0.5, seed=77)
    W, _, xq = make_case(fmt, N, K, "enc", 1500 + T.FMT[fmt], tokens=M)
    say("split-K gemm", fmt)
    xq_d, W_d, b_d = P.to_device(xq), P.to_device(W), P.to_device(bias)
    c0 = P.dev_gemm_nt(fmt, xq_d, W_d, b_d, M, N, K).cpu().numpy()
    ref = T.oracle_gemm_nt(fmt, xq, W, bias, M, N, K)
    assert T.norm_err(c0, ref) <= TOL
    for _ in range(3):
        assert np.array_equal(P.dev_gemm_nt(fmt, xq_d, W_d, b_d, M, N, K).cpu().numpy(), c0)
    # a second stream gets its own scratch
    import torch
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        c1 = P.dev_gemm_nt(fmt, xq_d, W_d, b_d, M, N, K)
    st.synchronize()
    assert np.array_equal(c1.cpu().numpy(), c0)


def test_gemm_mfma_q4_k_two_wave_groups_per_tile():
    """160 tiles and nine K-blocks: one tile per CU, so the launch gives every
    tile two groups of waves that take alternate K-blocks (five and four) and
    add their partial tiles in a fixed order.  The oracle on a sample of weight
    rows for every token, whole rows against the GEMV kernel for a few tokens,
    and the same bits on a second run."""
    M, N, K = 512, 2560, 2304
    W = T.synth_weights("q4_k", N, K, seed=5250)
    xf = T.normal(M * K, 0.0, 1.0, seed=5251)
    bias = T.normal(N, 0.0, 0.5, seed=5252)
    say("gemm mfma q4_k two wave groups")
    xq_d = P.dev_quantize(P.to_device(xf), "q8_k", rows=M)
    xq = xq_d.cpu().numpy()
    Wd, bd = P.to_device(W), P.to_device(bias)
    c = P.dev_gemm_nt("q4_k", xq_d, Wd, bd, M, N, K).cpu().numpy()
    rb = T.row_bytes("q4_k", K)
    rows = np.array([0, 1, 31, 32, 127, 128, 1279, 1280, 2558, 2559])
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    ref = T.oracle_gemm_nt("q4_k", xq, Wsub, np.ascontiguousarray(bias[rows]), M, len(rows), K)
    assert T.norm_err(c[:, rows], ref) <= TOL
    ab = T.row_bytes("q8_k", K)
    for t in (0, 63, 64, 300, 511):
        y = P.dev_gemm_nt("q4_k", P.to_device(xq[t * ab:(t + 1) * ab].copy()), Wd, bd, 1, N, K).cpu().numpy().reshape(-1)
        assert T.norm_err(c[t], y) <= 2e-6, t
    assert np.array_equal(P.dev_gemm_nt("q4_k", xq_d, Wd, bd, M, N, K).cpu().numpy(), c)


# ---- matrix-core GEMMs on seeded random shapes ---------------------------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
def test_gemm_mfma_random_shapes(fmt):
    """Ragged token counts, row counts that are no multiple of the 32-row wave
    slice or the 128-row tile, K from one block up, with and without bias and
    with a row pitch wider than N: every combination a tile edge can meet."""
    import torch
    rng = np.random.default_rng(20240 + T.FMT[fmt])
    lo = 65 if fmt == "q5_k" else 17
    for case in range(10):
        M = int(rng.integers(lo, 210))
        N = int(rng.integers(1, 300))
        K = int(rng.integers(1, 21)) * 32 if fmt == "q8_0" else int(rng.integers(1, 7)) * 256
        use_bias = bool(case & 1)
        ldc = N + int(rng.integers(0, 9)) if case % 3 == 0 else N
        W, _, xq = make_case(fmt, N, K, "enc" if case & 2 else "rand", 7000 + 31 * case + T.FMT[fmt], tokens=M)
        bias = T.normal(N, 0.0, 0.5, seed=case) if use_bias else None
        say("gemm mfma random", fmt, "M", M, "N", N, "K", K, "ldc", ldc, "bias", use_bias)
        ref = T.oracle_gemm_nt(fmt, xq, W, bias, M, N, K)
        xq_d, W_d = P.to_device(xq), P.to_device(W)
        b_d = P.to_device(bias) if use_bias else None
        c_d = torch.full((M * ldc,), 3.0, dtype=torch.float32, device="cuda")
        P.check(ckq.lib().ckq_gemm_nt_dev(P.FMT[fmt], P._dp(xq_d), P._dp(W_d), P._dp(b_d), P._dp(c_d), M, N, K, ldc,
                                          P._stream()), "ckq_gemm_nt_dev")
        c = c_d.cpu().numpy().reshape(M, ldc)
        assert T.norm_err(c[:, :N], ref) <= TOL, (fmt, M, N, K, ldc)
        assert np.all(c[:, N:] == 3.0), (fmt, M, N, K, ldc)         # nothing written beyond a row's N outputs


# ---- Q5_0 weights x Q8_0 activations ------------------------------------------------------------

def test_q5_0_subblock_dots_and_gemv_k_sweep():
    rows = 41
    for K in (32, 128, 512, 896, 1024, 2048, 4096, 8192, 10240):
        for kind in ("rand", "enc"):
            W, _, xq = make_case("q5_0", rows, K, kind, 60 + K)
            say("q5_0", kind, "rows", rows, "K", K)
            W_d, xq_d = P.to_device(W), P.to_device(xq)
            got = P.dev_subblock_dots("q5_0", W_d, xq_d, rows, K).cpu().numpy()
            assert np.array_equal(got, T.oracle_subdots("q5_0", W, xq, rows, K)), K
            y = P.dev_gemm_nt("q5_0", xq_d, W_d, None, 1, rows, K).cpu().numpy().reshape(-1)
            assert T.norm_err(y, T.oracle_gemv("q5_0", W, xq, rows, K)) <= TOL, (K, kind)


@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_q5_0_golden_fixture(kind):
    G = T.golden()
    M, K, TOK = (int(v) for v in G["shape"])
    W, xq = G["w_q5_0_" + kind], G["act_q80"]
    say("q5_0 golden", kind)
    y = P.gemv("q5_0", W, xq, M, K)
    c = P.gemm_nt("q5_0", xq, W, G["bias"], TOK, M, K)
    for build in ("avx2", "avx512"):
        assert T.norm_err(y, G["y_q5_0_%s_%s" % (kind, build)]) <= TOL
        assert T.norm_err(c, G["c_q5_0_%s_%s" % (kind, build)].reshape(TOK, M)) <= TOL
    s = np.zeros(1, np.float32)
    ckq.lib().vec_dot_q5_0_q8_0(K, T.ptr(s), T.ptr(W), T.ptr(xq))
    assert abs(float(s[0]) - float(G["s_q5_0_%s_vecdot" % kind][0])) <= TOL * np.abs(y).max()
    yp = np.zeros(M, np.float32)
    for ith in range(5):
        ckq.lib().gemv_q5_0_q8_0_parallel_simd(T.ptr(yp), T.ptr(W), T.ptr(xq), M, K, ith, 5)
    assert np.array_equal(yp, y)


def test_q5_0_row_and_token_counts():
    """Token tiles up to eight tokens; above that (forced here, this matrix is
    small) the blocks are rewritten as Q8_0 blocks and the Q8_0 matrix-core GEMM
    runs: the same bits as that GEMM on weights converted by the oracle."""
    K = 896
    for rows in (1, 3, 17, 64, 65, 257):
        W, _, xq = make_case("q5_0", rows, K, "rand", 11 * rows)
        say("q5_0 rows", rows)
        assert T.norm_err(P.gemv("q5_0", W, xq, rows, K), T.oracle_gemv("q5_0", W, xq, rows, K)) <= TOL, rows
    N = 77
    bias = T.normal(N, 0.0, 0.5, seed=8)
    for M in (1, 2, 5, 8, 9, 16, 17, 33, 130, 512):
        W, _, xq = make_case("q5_0", N, K, "enc", 310 + M, tokens=M)
        say("q5_0 gemm_nt tokens", M)
        ref = T.oracle_gemm_nt("q5_0", xq, W, bias, M, N, K)
        c = P.gemm_nt("q5_0", xq, W, bias, M, N, K)
        assert T.norm_err(c, ref) <= TOL, M
        if M > 8:
            w8 = np.zeros(len(W) // 22 * 34, np.uint8)
            T.oracle().orc_q5_0_to_q8_0(T.ptr(W), T.ptr(w8), ctypes.c_size_t(len(W) // 22))
            assert np.array_equal(P.gemm_nt("q8_0", xq, w8, bias, M, N, K), c), M


def test_fused_mlp_q5_0_gate_up_golden_case():
    G = T.golden()
    SEQ, ED, AED, ID, AID = (int(v) for v in G["mlp_shape"])
    say("fused mlp q5_0 gate/up golden")
    got = P.fused_mlp_swiglu_prefill_w1w2_quant(G["mlp_x"], G["mlp_w1_q5_0"], G["mlp_b1"], "q5_0", G["mlp_w2_q4_k"],
                                                G["mlp_b2"], "q4_k", SEQ, ED, AED, ID, AID)
    assert T.norm_err(got, G["mlp_out_q5_0w1_q4_k_avx2"].reshape(SEQ, AED)) <= TOL


# ---- automatic choice between the streaming kernel and the matrix cores --------------------------

@pytest.mark.parametrize("fmt,N,K,expect", [
    ("q4_k", 4096, 4096, {8: "stream", 9: "stream", 16: "stream", 17: "matrix"}),      # 9.4 MB: two passes stream
    ("q4_k", 11008, 4096, {8: "stream", 9: "matrix"}),                                  # 25 MB
    ("q6_k", 1024, 4096, {16: "stream", 40: "stream", 49: "matrix"}),                   # 3.4 MB
    ("q8_0", 4864, 896, {64: "stream", 72: "stream", 73: "matrix"}),                    # 4.6 MB, aligned-load streaming
    ("q8_0", 32000, 4096, {16: "stream", 17: "matrix"}),                                # 139 MB: two passes still stream
    ("q5_k", 4864, 1024, {64: "stream", 96: "stream", 100: "matrix"}),                  # 3.3 MB, 40 MB budget
    ("q5_0", 896, 896, {48: "stream", 57: "matrix"}),                                   # below the 3 MB floor
])
def test_gemm_automatic_kernel_choice(fmt, N, K, expect):
    """With the default policy the library picks the kernel by token count and
    weight size.  Each result matches the oracle on a sample of rows, and equals
    bit for bit what the kernel it should have picked gives when forced."""
    L = ckq.lib()
    W = T.random_blocks(fmt, N * (K // T.ELEMS[fmt]), 4242)
    Wd = P.to_device(W)
    rb = T.row_bytes(fmt, K)
    rows = np.array([0, 1, N // 2, N - 1])
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    for M, which in expect.items():
        say("automatic kernel choice", fmt, N, K, M, which)
        xq = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 500 + M), T.act_fmt(fmt), rows=M)
        xd = P.to_device(xq)
        L.ckq_set_gemm_policy(0)
        auto = P.dev_gemm_nt(fmt, xd, Wd, None, M, N, K).cpu().numpy()
        assert T.norm_err(auto[:, rows], T.oracle_gemm_nt(fmt, xq, Wsub, None, M, len(rows), K)) <= TOL, M
        L.ckq_set_gemm_policy(1 if which == "matrix" else 2)
        forced = P.dev_gemm_nt(fmt, xd, Wd, None, M, N, K).cpu().numpy()
        L.ckq_set_gemm_policy(0)
        assert np.array_equal(auto, forced), (M, which)


# ---- sequences: independent entries of one shape share a launch ----------------------------------

@pytest.mark.parametrize("fmt,N,K", [("q4_k", 384, 1024), ("q6_k", 200, 512), ("q8_0", 130, 896), ("q5_k", 96, 768)])
def test_matmul_sequence_groups_independent_entries(fmt, N, K):
    """Q/K/V-like entries (one input, separate weights and outputs, K and V
    narrower than Q) and a pair with separate inputs go out as grouped launches
    at one token; every output has the bits of the same matmul launched alone,
    with and without biases, for one and several tokens, and the oracle's
    values."""
    import torch
    Ns = [N, N // 4 + 1, N // 4 + 1, N, N + 5, 2 * N]
    for M in (1, 3, 8):
        Ws = [T.random_blocks(fmt, Ns[i] * (K // T.ELEMS[fmt]), 700 + i) for i in range(6)]
        xs = [T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 800 + i), T.act_fmt(fmt), rows=M) for i in range(2)]
        bias = [T.normal(Ns[i], 0.0, 0.5, seed=900 + i) if i % 2 else None for i in range(6)]
        Wd = [P.to_device(w) for w in Ws]
        xd = [P.to_device(x) for x in xs]
        bd = [None if b is None else P.to_device(b) for b in bias]
        inp = [0, 0, 0, 1, 0, 1]                       # entries 0-2 share an input; 3-5 alternate
        outs = [torch.full((M * Ns[i],), 7.0, dtype=torch.float32, device="cuda") for i in range(6)]
        say("sequence grouping", fmt, M)
        P.dev_matmul_sequence([(fmt, xd[inp[i]], Wd[i], bd[i], outs[i], M, Ns[i], K) for i in range(6)])
        for i in range(6):
            alone = P.dev_gemm_nt(fmt, xd[inp[i]], Wd[i], bd[i], M, Ns[i], K).cpu().numpy()
            got = outs[i].cpu().numpy().reshape(M, Ns[i])
            assert np.array_equal(got, alone), (M, i)
            assert T.norm_err(got, T.oracle_gemm_nt(fmt, xs[inp[i]], Ws[i], bias[i], M, Ns[i], K)) <= TOL, (M, i)


def test_matmul_sequence_keeps_order_where_entries_depend():
    """Entries that write what a later entry reads, or write the same output,
    stay separate launches in list order: the bytes equal those of the same
    entries issued one call at a time."""
    import torch
    fmt, N, K, M = "q4_k", 1168, 1024, 1
    W1 = P.to_device(T.random_blocks(fmt, N * (K // 256), 31))
    W2 = P.to_device(T.random_blocks(fmt, N * (K // 256), 32))
    x = P.to_device(T.oracle_quantize(T.normal(K, 0.0, 1.0, 33), "q8_k"))
    say("sequence with dependent entries")

    def run(seq_call):
        a = torch.zeros(N, dtype=torch.float32, device="cuda")
        b = torch.zeros(N, dtype=torch.float32, device="cuda")
        ops = [(fmt, x, W1, None, a, M, N, K),
               (fmt, a, W2, None, b, M, N, K),      # reads the first 1168 bytes of `a` as a Q8_K row
               (fmt, x, W2, None, b, M, N, K),      # same output as the entry before: the last one wins
               (fmt, x, W1, None, a, M, N, K)]      # and `a` again
        if seq_call:
            P.dev_matmul_sequence(ops)
        else:
            for o in ops:
                P.dev_matmul_sequence([o])
        torch.cuda.synchronize()
        return a.cpu().numpy().view(np.uint32), b.cpu().numpy().view(np.uint32)

    a1, b1 = run(True)
    a2, b2 = run(False)
    assert np.array_equal(a1, a2) and np.array_equal(b1, b2)
    ref = P.dev_gemm_nt(fmt, x, W2, None, M, N, K).cpu().numpy().reshape(-1).view(np.uint32)
    assert np.array_equal(b1, ref)


def test_host_inputs_stored_straight_into_device_memory_are_never_stale():
    """Host-pointer calls copy small inputs with CPU stores into a device buffer the
    next kernel reads (no upload launch).  3000 calls in a row, each with a
    different activation vector of a different length and, every other call, a
    bias: every result has the bits the device-pointer path gives for the same
    inputs, so no call has read an earlier call's bytes."""
    import torch
    rng = np.random.default_rng(4711)
    N = 384
    Ks = [256, 512, 1024, 2048]
    Wh = {K: T.synth_weights("q4_k", N, K, seed=900 + K) for K in Ks}
    Wd = {K: P.to_device(Wh[K]) for K in Ks}
    pool = {K: [T.oracle_quantize(T.normal(K, 0.0, 1.0 + 0.1 * i, seed=1000 * K + i), "q8_k") for i in range(24)] for K in Ks}
    biases = [T.normal(N, 0.0, 1.0, seed=77 + i) for i in range(4)]
    want = {}
    for K in Ks:
        for i, xq in enumerate(pool[K]):
            for bi in (-1, 0, 1, 2, 3):
                b = None if bi < 0 else P.to_device(biases[bi])
                want[(K, i, bi)] = P.dev_gemm_nt("q4_k", P.to_device(xq), Wd[K], b, 1, N, K).cpu().numpy().reshape(-1)
    torch.cuda.synchronize()
    say("3000 host-pointer calls with changing inputs")
    bad = 0
    for it in range(3000):
        K = Ks[int(rng.integers(len(Ks)))]
        i = int(rng.integers(24))
        bi = int(rng.integers(4)) if it & 1 else -1
        xq = pool[K][i].copy()                      # a fresh host address most of the time
        got = P.gemm_nt("q4_k", xq, Wh[K], None if bi < 0 else biases[bi], 1, N, K).reshape(-1)
        bad += int(not np.array_equal(got, want[(K, i, bi)]))
    assert bad == 0, "%d of 3000 calls read stale inputs" % bad
