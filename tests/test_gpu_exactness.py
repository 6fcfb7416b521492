"""GPU tests of what is bit-exact on the path and of the shapes the benchmark
times: integer sub-block dots taken from the PRODUCTION instantiations of the
streaming kernel (staged activations, two rows per wave, 512-thread blocks,
token tiles, grouped launches), the integer block sums of the four matrix-core
GEMMs, fp16 scales at the ends of their range, and parity at the benchmark's
batched-decode and grouped-launch shapes.  Expected integers come from NumPy
decoders written from the format definitions (tests/ckq_testlib.py), not from
the oracle's C code."""
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


def say(*a):
    print(*a)
    sys.stdout.flush()


@pytest.fixture(scope="module", autouse=True)
def _lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    L = ckq.lib()
    assert L.ckq_init() == 0
    L.ckq_set_gemm_policy(0)
    yield L
    L.ckq_weights_clear()


def rand_case(fmt, rows, K, seed, tokens=1):
    W = T.random_blocks(fmt, rows * (K // T.ELEMS[fmt]), seed)
    xq = T.oracle_quantize(T.normal(tokens * K, 0.0, 1.0, seed + 1000), T.act_fmt(fmt), rows=tokens)
    return W, xq


def np_subdots_tokens(fmt, W, xq, rows, K, tokens):
    xb = T.row_bytes(T.act_fmt(fmt), K)
    return np.stack([T.np_subdots(fmt, W, xq[t * xb:(t + 1) * xb], rows, K) for t in range(tokens)])


# ---- streaming kernel: integer dots from the instantiations that production launches --------------

# (format, rows, K, tokens): what each shape selects
PRODUCTION_SHAPES = [
    ("q4_k", 300, 4096, 1),      # one row per wave, 256-thread blocks, staged activations (the headline instantiation)
    ("q4_k", 16500, 4096, 1),    # more than 16 384 waves: two rows per wave
    ("q4_k", 2100, 8192, 1),     # rows longer than one pass, >= 2048 rows: 512-thread blocks
    ("q6_k", 8200, 11008, 1),    # long rows, >= 8192 rows: two rows per slot (K = 11008: three positions per lane)
    ("q6_k", 16500, 4096, 1),
    ("q5_k", 900, 4864, 1),      # the small model's down projection
    ("q8_0", 16500, 896, 1),     # paired-block trait, two rows per wave
    ("q8_0", 700, 4096, 1),
    ("q4_k", 333, 4096, 2), ("q4_k", 333, 4096, 3), ("q4_k", 333, 4096, 8),
    ("q5_k", 129, 1024, 4), ("q5_k", 129, 1024, 8),
    ("q6_k", 200, 4096, 2), ("q6_k", 200, 2048, 7),
    ("q8_0", 515, 896, 2), ("q8_0", 515, 896, 4), ("q8_0", 515, 896, 8),
]


@pytest.mark.parametrize("fmt,rows,K,tokens", PRODUCTION_SHAPES)
def test_production_instantiation_subblock_dots_bit_exact(fmt, rows, K, tokens):
    W, xq = rand_case(fmt, rows, K, 11 * rows + K + tokens, tokens)
    say("production dump", fmt, rows, K, "tokens", tokens)
    got = P.dev_subblock_dots_tokens(fmt, P.to_device(W), P.to_device(xq), rows, K, tokens).cpu().numpy()
    want = np_subdots_tokens(fmt, W, xq, rows, K, tokens)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("fmt,rows,K", [("q4_k", [520, 130, 130], 4096), ("q4_k", [1100, 1100], 4096),
                                        ("q5_k", [896, 128, 128], 1024), ("q6_k", [300, 300, 77, 5], 2048),
                                        ("q8_0", [640, 64], 896)])
@pytest.mark.parametrize("tokens", [1, 8])
def test_grouped_launch_subblock_dots_bit_exact(fmt, rows, K, tokens):
    """One grouped launch (Q/K/V- and gate/up-like problems of unequal row
    counts): the integer dots of every problem equal the brute-force ones."""
    n = len(rows)
    Ws = [T.random_blocks(fmt, r * (K // T.ELEMS[fmt]), 500 + i) for i, r in enumerate(rows)]
    xs = [T.oracle_quantize(T.normal(tokens * K, 0.0, 1.0, 600 + (i % 2)), T.act_fmt(fmt), rows=tokens) for i in range(n)]
    say("grouped dump", fmt, rows, K, tokens)
    got = P.dev_subblock_dots_group(fmt, [P.to_device(w) for w in Ws], [P.to_device(x) for x in xs], rows, K,
                                    tokens).cpu().numpy()
    for g in range(n):
        want = np_subdots_tokens(fmt, Ws[g], xs[g], rows[g], K, tokens)
        assert np.array_equal(got[g][:, :rows[g]], want), g
        assert not got[g][:, rows[g]:].any()


def test_product_library_has_no_dump_kernels():
    """The integer dumps are test infrastructure: the shipped library answers
    their entry points with CKQ_ENODUMP (-6) and enqueues nothing; the test
    build of the same sources (libckernel_quant_hip_dump.so) runs them."""
    import torch
    L = ckq.lib()
    W = P.to_device(T.synth_weights("q4_k", 64, 256, seed=1))
    x = P.to_device(T.oracle_quantize(T.normal(256, 0.0, 1.0, 2), "q8_k"))
    out = torch.full((64 * 8,), 77, dtype=torch.int32, device="cuda")
    assert L.ckq_subblock_dots_dev(P.FMT["q4_k"], P._dp(out), P._dp(W), P._dp(x), 64, 256, P._stream()) == -6
    c = torch.zeros(64, dtype=torch.float32, device="cuda")
    assert L.ckq_gemm_block_sums_dev(P.FMT["q4_k"], P._dp(x), P._dp(W), None, P._dp(c), P._dp(out), 1, 64, 256, P._stream()) == -6
    torch.cuda.synchronize()
    assert (out == 77).all()
    assert b"dump" in L.ckq_error_string(-6)
    assert np.array_equal(P.dev_subblock_dots("q4_k", W, x, 64, 256).cpu().numpy(),
                          T.oracle_subdots("q4_k", T.synth_weights("q4_k", 64, 256, seed=1), x.cpu().numpy(), 64, 256))


# ---- matrix-core GEMMs: integer block sums ----------------------------------------------------------

def np_block_sums(fmt, W, A, M, N, K):
    """[M, N, nblk, per] from the format definitions (int64 arithmetic)."""
    if fmt == "q8_0":
        wq = T.np_decode_q8_0(W)["q"].reshape(N, K // 32, 32).astype(np.int64)
        xq = T.np_decode_q8_0(A)["q"].reshape(M, K // 32, 32).astype(np.int64)
        return np.einsum("njk,tjk->tnj", wq, xq)[..., None]
    nb = K // 256
    x = T.np_decode_q8_k(A)
    xq = x["q"].reshape(M, nb, 256).astype(np.int64)
    if fmt == "q6_k":
        d = T.np_decode_q6_k(W)
        ws = (d["q"].reshape(N, nb, 16, 16) * d["sc"].reshape(N, nb, 16, 1)).reshape(N, nb, 256).astype(np.int64)
        return np.einsum("nbk,tbk->tnb", ws, xq)[..., None]
    d = (T.np_decode_q4_k if fmt == "q4_k" else T.np_decode_q5_k)(W)
    sc = d["sc"].reshape(N, nb, 8).astype(np.int64)
    mn = d["mn"].reshape(N, nb, 8).astype(np.int64)
    ws = (d["q"].reshape(N, nb, 8, 32) * sc[..., None]).reshape(N, nb, 256).astype(np.int64)
    i1 = np.einsum("nbk,tbk->tnb", ws, xq)
    pairs = x["bsums"].reshape(M, nb, 8, 2).sum(axis=3).astype(np.int64)      # STORED bsums
    i2 = np.einsum("nbj,tbj->tnb", mn, pairs)
    return np.stack([i1, i2], axis=-1)


GEMM_DUMP_SHAPES = {
    "q4_k": [(70, 200, 1024), (130, 384, 2048), (33, 128, 256), (64, 130, 4096), (520, 260, 512)],
    # K = 768 and 1536: 3 and 6 K-blocks, the exit of the three-stage K loops after a whole round of stages
    "q5_k": [(70, 200, 1024), (66, 96, 512), (130, 333, 2048), (40, 160, 768), (70, 130, 1536)],
    "q6_k": [(70, 200, 1024), (130, 1100, 512), (33, 128, 256), (140, 384, 2048),    # 64- and 128-token tiles
             (40, 160, 768), (140, 130, 1536), (70, 96, 2304)],
    "q8_0": [(70, 200, 896), (130, 333, 160), (33, 128, 32), (64, 96, 1024)],
}


@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
def test_gemm_mfma_integer_block_sums_bit_exact(fmt):
    """I1 / I2 (Q4_K, Q5_K), the Q6_K block sum and the Q8_0 block dots of the
    matrix-core kernels, per (token, row, block), against brute force; the fp32
    result of the dump build equals the production build's bit for bit."""
    L = ckq.lib()
    for M, N, K in GEMM_DUMP_SHAPES[fmt]:
        W, A = rand_case(fmt, N, K, 3 * M + N + K, tokens=M)
        say("gemm block sums", fmt, M, N, K)
        Ad, Wd = P.to_device(A), P.to_device(W)
        c, sums = P.dev_gemm_block_sums(fmt, Ad, Wd, None, M, N, K)
        want = np_block_sums(fmt, W, A, M, N, K)
        assert np.array_equal(sums.cpu().numpy().astype(np.int64), want), (M, N, K)
        L.ckq_set_gemm_policy(1)
        try:
            prod = P.dev_gemm_nt(fmt, Ad, Wd, None, M, N, K).cpu().numpy() if M > 8 else None
        finally:
            L.ckq_set_gemm_policy(0)
        if prod is not None:
            assert np.array_equal(c.cpu().numpy(), prod), (M, N, K)
        assert T.norm_err(c.cpu().numpy(), T.oracle_gemm_nt(fmt, A, W, None, M, N, K)) <= TOL


def test_gemm_mfma_block_sums_extremes():
    """Saturating operands: every nibble 15, every scale and min 63, every
    activation -128 / 127 and the largest stored bsums: the integer sums reach
    their bounds (|I1| = 256 * 945 * 128) and stay exact."""
    M, N, K = 64, 128, 512
    nb = K // 256
    W = np.zeros((N * nb, 144), np.uint8)
    W[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    W[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    W[:, 4:16] = 0xff
    W[:, 16:] = 0xff
    A = np.zeros((M * nb, 292), np.uint8)
    A[:, 0:4] = np.frombuffer(np.float32(0.05).tobytes(), np.uint8)
    q = np.where((np.arange(M * nb)[:, None] + 0 * np.arange(256)[None, :]) % 2 == 0, -128, 127).astype(np.int8)
    A[:, 4:260] = q.view(np.uint8)
    A[:, 260:292] = q.reshape(-1, 16, 16).sum(axis=2).astype(np.int16).view(np.uint8).reshape(-1, 32)
    W, A = W.reshape(-1), A.reshape(-1)
    c, sums = P.dev_gemm_block_sums("q4_k", P.to_device(A), P.to_device(W), None, M, N, K)
    want = np_block_sums("q4_k", W, A, M, N, K)
    assert np.abs(want[..., 0]).max() >= 63 * 15 * 127 * 128
    assert np.array_equal(sums.cpu().numpy().astype(np.int64), want)
    assert T.norm_err(c.cpu().numpy(), T.oracle_gemm_nt("q4_k", A, W, None, M, N, K)) <= TOL


# ---- fp16 scales at the ends of their range ----------------------------------------------------------

def _set_f16(blocks, off, bits):
    blocks[:, off] = bits & 0xff
    blocks[:, off + 1] = bits >> 8


@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
def test_fp16_scales_subnormal_and_max_finite(fmt):
    """Rows whose fp16 block scales are subnormal (0x0001, 0x03ff), the smallest
    normal, the largest finite (0x7bff) and negative: the device's half->float
    conversion keeps subnormals, like the reference's (ckernel_quant.h:265-294)."""
    K = 1024
    nbr = K // T.ELEMS[fmt]
    patterns = [0x0001, 0x03ff, 0x0400, 0x7bff, 0x8001, 0xfbff, 0x3c00, 0x0200]
    rows = len(patterns) * 5
    W = T.random_blocks(fmt, rows * nbr, 77).reshape(rows * nbr, T.BLK[fmt]).copy()
    d_off = {"q4_k": 0, "q5_k": 0, "q6_k": 208, "q8_0": 0}[fmt]
    for i in range(rows):
        blk = W[i * nbr:(i + 1) * nbr]
        _set_f16(blk, d_off, patterns[i % len(patterns)])
        if fmt in ("q4_k", "q5_k"):
            _set_f16(blk, 2, patterns[(i // len(patterns) + i) % len(patterns)])
    W = W.reshape(-1)
    for tokens in (1, 4):
        xq = T.oracle_quantize(T.normal(tokens * K, 0.0, 1.0, 78), T.act_fmt(fmt), rows=tokens)
        say("fp16 scale range", fmt, tokens)
        got = P.dev_gemm_nt(fmt, P.to_device(xq), P.to_device(W), None, tokens, rows, K).cpu().numpy()
        want = T.oracle_gemm_nt(fmt, xq, W, None, tokens, rows, K)
        assert np.all(np.isfinite(want))
        # pattern by pattern (five rows each): a subnormal-scaled row must not be judged
        # against the largest row of the matrix
        for p in range(len(patterns)):
            rs = np.arange(p, rows, len(patterns))
            den = max(np.abs(want[:, rs]).max(), 1e-30)
            assert np.abs(got[:, rs] - want[:, rs]).max() / den <= TOL, hex(patterns[p])
            assert np.abs(got[:, rs]).max() > 0, "a subnormal scale was flushed to zero"
    # the prefill kernels read the same scales
    L = ckq.lib()
    M = 40
    A = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 79), T.act_fmt(fmt), rows=M)
    L.ckq_set_gemm_policy(1)
    try:
        got = P.dev_gemm_nt(fmt, P.to_device(A), P.to_device(W), None, M, rows, K).cpu().numpy()
    finally:
        L.ckq_set_gemm_policy(0)
    want = T.oracle_gemm_nt(fmt, A, W, None, M, rows, K)
    for p in range(len(patterns)):
        rs = np.arange(p, rows, len(patterns))
        den = max(np.abs(want[:, rs]).max(), 1e-30)
        assert np.abs(got[:, rs] - want[:, rs]).max() / den <= TOL, ("gemm", hex(patterns[p]))


def test_fp16_scale_inf_propagates():
    """An infinite block scale gives a non-finite output in that row only, as on the CPU."""
    fmt, K, rows = "q4_k", 512, 6
    W = T.random_blocks(fmt, rows * 2, 5).reshape(rows * 2, 144).copy()
    _set_f16(W[4:6], 0, 0x7c00)
    W = W.reshape(-1)
    xq = T.oracle_quantize(T.normal(K, 0.0, 1.0, 6), "q8_k")
    got = P.dev_gemm_nt(fmt, P.to_device(xq), P.to_device(W), None, 1, rows, K).cpu().numpy().reshape(-1)
    want = T.oracle_gemv(fmt, W, xq, rows, K)
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    assert not np.isfinite(got[2]) and np.isfinite(got[[0, 1, 3, 4, 5]]).all()


# ---- what the benchmark times is what is checked -------------------------------------------------------

def _sampled_rows(N, n=96, seed=3):
    r = np.unique(np.concatenate([np.arange(8), np.arange(N - 8, N),
                                  np.random.default_rng(seed).integers(0, N, n)]))
    return r


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_q8_0_lm_head_151936x896_batched_decode(M):
    """The small model's LM head at the benchmark's batched-decode sizes: every
    token, sampled rows against the oracle; all rows through two size-independent
    properties (run-to-run identical bits; each token equals its own GEMV)."""
    import torch
    fmt, N, K = "q8_0", 151936, 896
    W = T.synth_weights(fmt, N, K, seed=2100)
    xq = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 43), "q8_0", rows=M)
    Wd, xd = P.to_device(W), P.to_device(xq)
    say("Q8_0 LM head 151936x896 M =", M)
    c = P.dev_gemm_nt(fmt, xd, Wd, None, M, N, K).cpu().numpy()
    rows = _sampled_rows(N)
    rb = T.row_bytes(fmt, K)
    Wsub = np.ascontiguousarray(W.reshape(N, rb)[rows]).reshape(-1)
    assert T.norm_err(c[:, rows], T.oracle_gemm_nt(fmt, xq, Wsub, None, M, len(rows), K)) <= TOL
    again = P.dev_gemm_nt(fmt, xd, Wd, None, M, N, K).cpu().numpy()
    assert np.array_equal(c, again)
    xb = T.row_bytes("q8_0", K)
    for t in range(M):
        one = P.dev_gemm_nt(fmt, P.to_device(xq[t * xb:(t + 1) * xb]), Wd, None, 1, N, K).cpu().numpy().reshape(-1)
        assert T.norm_err(c[t], one) <= 2e-6, t
    torch.cuda.synchronize()


GROUPS = [("q4_k", [4096, 4096, 4096], 4096), ("q4_k", [11008, 11008], 4096), ("q5_k", [896, 128, 128], 1024),
          ("q5_k", [4864, 4864], 1024)]


@pytest.mark.parametrize("fmt,Ns,K", GROUPS)
@pytest.mark.parametrize("M", [1, 8])
def test_grouped_launch_at_benchmark_shapes(fmt, Ns, K, M):
    """Q+K+V of a 7B layer, its gate+up, and the small model's Q/K/V and gate/up
    as ONE grouped launch each: the bits of the same matmuls launched alone, and
    the oracle's values on sampled rows."""
    import torch
    n = len(Ns)
    Ws = [T.synth_weights(fmt, Ns[i], K, seed=1000 + i) for i in range(n)]
    xq = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 31), "q8_k", rows=M)
    Wd, xd = [P.to_device(w) for w in Ws], P.to_device(xq)
    outs = [torch.full((M * Ns[i],), 7.0, dtype=torch.float32, device="cuda") for i in range(n)]
    say("grouped launch", fmt, Ns, K, "M", M)
    P.dev_matmul_sequence([(fmt, xd, Wd[i], None, outs[i], M, Ns[i], K) for i in range(n)])
    rb = T.row_bytes(fmt, K)
    for i in range(n):
        alone = P.dev_gemm_nt(fmt, xd, Wd[i], None, M, Ns[i], K).cpu().numpy()
        got = outs[i].cpu().numpy().reshape(M, Ns[i])
        assert np.array_equal(got, alone), i
        rows = _sampled_rows(Ns[i], 64, seed=i)
        Wsub = np.ascontiguousarray(Ws[i].reshape(Ns[i], rb)[rows]).reshape(-1)
        assert T.norm_err(got[:, rows], T.oracle_gemm_nt(fmt, xq, Wsub, None, M, len(rows), K)) <= TOL, i


def test_sequence_group_whose_tile_exceeds_lds_is_issued_separately():
    """Three independent entries with M = 5 tokens of K = 8192: the token tile
    (eight rows of activations) does not fit 64 KB of LDS, so the entries go out
    as separate launches instead of failing."""
    import torch
    fmt, N, K, M = "q4_k", 200, 8192, 5
    Ws = [T.random_blocks(fmt, N * (K // 256), 40 + i) for i in range(3)]
    xq = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 44), "q8_k", rows=M)
    Wd, xd = [P.to_device(w) for w in Ws], P.to_device(xq)
    outs = [torch.full((M * N,), 7.0, dtype=torch.float32, device="cuda") for _ in range(3)]
    P.dev_matmul_sequence([(fmt, xd, Wd[i], None, outs[i], M, N, K) for i in range(3)])
    for i in range(3):
        got = outs[i].cpu().numpy().reshape(M, N)
        assert T.norm_err(got, T.oracle_gemm_nt(fmt, xq, Ws[i], None, M, N, K)) <= TOL, i
    # Q8_0 at 9 K bytes per token: M = 8, K = 8192 exceeds it as well
    fmt, K, M = "q8_0", 8192, 8
    Ws = [T.random_blocks(fmt, N * (K // 32), 50 + i) for i in range(2)]
    xq = T.oracle_quantize(T.normal(M * K, 0.0, 1.0, 54), "q8_0", rows=M)
    Wd, xd = [P.to_device(w) for w in Ws], P.to_device(xq)
    outs = [torch.full((M * N,), 7.0, dtype=torch.float32, device="cuda") for _ in range(2)]
    P.dev_matmul_sequence([(fmt, xd, Wd[i], None, outs[i], M, N, K) for i in range(2)])
    for i in range(2):
        assert T.norm_err(outs[i].cpu().numpy().reshape(M, N), T.oracle_gemm_nt(fmt, xq, Ws[i], None, M, N, K)) <= TOL, i


def test_sequence_with_producer_steps():
    """A decode layer's chain as ONE C call: RMSNorm->Q8_K, Q/K/V (one grouped
    launch), Q8_K of the attention output, O, RMSNorm->Q8_K, gate/up (grouped),
    SiLU(gate)*up->Q8_K, down.  Every buffer has the bits of the same steps issued
    one call at a time; the producers are bit-exact with the oracle."""
    import torch
    D, F, KV, M = 1024, 2816, 256, 1
    x = T.normal(M * D, 0.0, 1.0, 91)
    gam1, gam2 = T.normal(D, 1.0, 0.2, seed=92), T.normal(D, 1.0, 0.2, seed=93)
    Wq, Wk, Wv = (T.synth_weights("q4_k", n, D, seed=94 + i) for i, n in enumerate((D, KV, KV)))
    Wo = T.synth_weights("q4_k", D, D, seed=97)
    Wg, Wu = T.synth_weights("q4_k", F, D, seed=98), T.synth_weights("q4_k", F, D, seed=99)
    Wd = T.synth_weights("q6_k", D, F, seed=100)
    dev = {k: P.to_device(v) for k, v in dict(x=x, g1=gam1, g2=gam2, Wq=Wq, Wk=Wk, Wv=Wv, Wo=Wo, Wg=Wg, Wu=Wu, Wd=Wd).items()}
    f32 = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")
    u8 = lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda")

    def buffers():
        return dict(xq=u8(T.row_bytes("q8_k", D)), q=f32(D), k=f32(KV), v=f32(KV), aq=u8(T.row_bytes("q8_k", D)), o=f32(D),
                    fq=u8(T.row_bytes("q8_k", D)), g=f32(F), u=f32(F), hq=u8(T.row_bytes("q8_k", F)), y=f32(D))

    def steps(b):
        return [("rmsnorm_q8_k", dev["x"], dev["g1"], b["xq"], M, D, D, 1e-5),
                ("q4_k", b["xq"], dev["Wq"], None, b["q"], M, D, D),
                ("q4_k", b["xq"], dev["Wk"], None, b["k"], M, KV, D),
                ("q4_k", b["xq"], dev["Wv"], None, b["v"], M, KV, D),
                ("quantize_q8_k", b["q"], None, b["aq"], M, D),              # stands in for the attention output
                ("q4_k", b["aq"], dev["Wo"], None, b["o"], M, D, D),
                ("rmsnorm_q8_k", b["o"], dev["g2"], b["fq"], M, D, D, 1e-5),
                ("q4_k", b["fq"], dev["Wg"], None, b["g"], M, F, D),
                ("q4_k", b["fq"], dev["Wu"], None, b["u"], M, F, D),
                ("swiglu_q8_k", b["g"], b["u"], b["hq"], M, F, F),
                ("q6_k", b["hq"], dev["Wd"], None, b["y"], M, D, F)]

    say("decode chain with producer steps, one call")
    one = buffers()
    P.dev_matmul_sequence(steps(one), repeat=2)
    sep = buffers()
    for st in steps(sep):
        P.dev_matmul_sequence([st])
    torch.cuda.synchronize()
    for name in one:
        assert torch.equal(one[name], sep[name]), name
    # producers against the oracle, matmuls against the oracle on the device's own activations
    xq = one["xq"].cpu().numpy()
    want = np.zeros_like(xq)
    T.oracle().orc_rmsnorm_q8_k_fused(T.ptr(x), T.ptr(gam1), T.ptr(want), M, D, D, ctypes.c_float(1e-5))
    assert np.array_equal(xq, want)
    assert np.array_equal(one["aq"].cpu().numpy(), T.oracle_quantize(one["q"].cpu().numpy(), "q8_k"))
    assert T.norm_err(one["q"].cpu().numpy(), T.oracle_gemv("q4_k", Wq, xq, D, D)) <= TOL
    assert T.norm_err(one["y"].cpu().numpy(), T.oracle_gemv("q6_k", Wd, one["hq"].cpu().numpy(), D, F)) <= TOL


# ---- producer steps in a sequence, one activation buffer reused ------------------------------------------

def test_sequence_steps_reuse_one_activation_buffer():
    """Consecutive (quantizer, matmul) pairs of one sequence call write DIFFERENT
    activations into the same Q8_K buffer (as every layer of a model does), for
    the three producers and one to eight tokens: each matmul sees its own
    producer's blocks; the producers are bit-exact with the oracle."""
    import torch
    f32 = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")
    N, K, R = 3000, 4096, 4
    W = P.to_device(T.synth_weights("q4_k", N, K, seed=17))
    gam = T.normal(K, 1.0, 0.2, seed=18)
    gam_t = P.to_device(gam)
    for M in (1, 4, 8):
        xs = [T.normal(M * K, 0.0, 1.0 + r, seed=300 + r) for r in range(R)]
        xs_t = [P.to_device(x) for x in xs]
        xq = torch.zeros(M * T.row_bytes("q8_k", K), dtype=torch.uint8, device="cuda")
        ys = [f32(M * N) for _ in range(R)]
        kinds = ["quantize_q8_k", "rmsnorm_q8_k", "swiglu_q8_k", "quantize_q8_k"]
        steps = []
        for r in range(R):
            pro = {"quantize_q8_k": ("quantize_q8_k", xs_t[r], None, xq, M, K),
                   "rmsnorm_q8_k": ("rmsnorm_q8_k", xs_t[r], gam_t, xq, M, K, K, 1e-5),
                   "swiglu_q8_k": ("swiglu_q8_k", xs_t[r], xs_t[(r + 1) % R], xq, M, K, K)}[kinds[r]]
            steps += [pro, ("q4_k", xq, W, None, ys[r], M, N, K)]
        say(f"producer steps sharing one activation buffer M={M}")
        P.dev_matmul_sequence(steps, repeat=2)
        torch.cuda.synchronize()
        for r in range(R):
            if kinds[r] == "quantize_q8_k":
                want_q = T.oracle_quantize(xs[r], "q8_k", rows=M)
            elif kinds[r] == "rmsnorm_q8_k":
                want_q = np.zeros(M * T.row_bytes("q8_k", K), np.uint8)
                T.oracle().orc_rmsnorm_q8_k_fused(T.ptr(xs[r]), T.ptr(gam), T.ptr(want_q), M, K, K, ctypes.c_float(1e-5))
            else:
                want_q = P.dev_swiglu_q8_k(xs_t[r], xs_t[(r + 1) % R], M, K, K).cpu().numpy()
            want = P.dev_gemm_nt("q4_k", P.to_device(want_q), W, None, M, N, K).view(-1)
            assert torch.equal(ys[r], want), (M, r)


def test_sequence_with_fp32_activation_entries():
    """A sequence entry tagged CKQ_ACT_F32 computes what ckq_gemm_nt_f32act_dev
    computes, between ordinary entries."""
    import torch
    N, K, M = 300, 1024, 2
    x = T.normal(M * K, 0.0, 1.0, seed=81)
    x_t = P.to_device(x)
    for fmt in ("q4_k", "q6_k", "q8_0"):
        W = P.to_device(T.synth_weights(fmt, N, K, seed=82))
        xq = P.dev_quantize(x_t, T.act_fmt(fmt), rows=M)
        y0 = torch.zeros(M * N, dtype=torch.float32, device="cuda")
        y1, y2 = torch.zeros_like(y0), torch.zeros_like(y0)
        say("sequence with fp32-activation entry", fmt)
        P.dev_matmul_sequence([(fmt, xq, W, None, y0, M, N, K), (fmt + "+f32", x_t, W, None, y1, M, N, K),
                               (fmt, xq, W, None, y2, M, N, K)])
        torch.cuda.synchronize()
        assert torch.equal(y1, P.dev_gemm_nt_f32act(fmt, x_t, W, None, M, N, K).view(-1))
        assert torch.equal(y0, y2) and torch.equal(y0, P.dev_gemm_nt(fmt, xq, W, None, M, N, K).view(-1))


# ---- grouped matrix-core launches (Q/K/V, gate/up at prefill sizes) ------------------------------------

@pytest.mark.parametrize("fmt,K", [("q4_k", 1024), ("q5_k", 1024), ("q6_k", 1024), ("q8_0", 512)])
def test_grouped_prefill_launch_equals_single_launches(fmt, K):
    """Three matrices of different, ragged heights against the same 500 tokens as
    consecutive sequence entries go out as ONE matrix-core launch (168 tiles); every
    output has the bits of the single-matrix launch (K is short enough that no
    single launch is split along K), with and without bias, in a padded C."""
    import torch
    L = ckq.lib()
    M, Ns = 500, [1536, 640, 392]
    x = P.to_device(T.normal(M * K, 0.0, 1.0, seed=301))
    xq = P.dev_quantize(x, T.act_fmt(fmt), rows=M)
    Ws = [P.to_device(T.synth_weights(fmt, n, K, seed=302 + i)) for i, n in enumerate(Ns)]
    bs = [None, P.to_device(T.normal(Ns[1], 0.0, 1.0, seed=310)), None]
    L.ckq_set_gemm_policy(1)
    try:
        ldc = [n + 8 for n in Ns]
        ys = [torch.full((M * l,), 7.0, dtype=torch.float32, device="cuda") for l in ldc]
        say("grouped prefill launch", fmt, M, Ns, K)
        P.dev_matmul_sequence([(fmt, xq, W, b, y, M, n, K, l) for W, b, y, n, l in zip(Ws, bs, ys, Ns, ldc)])
        torch.cuda.synchronize()
        for W, b, y, n, l in zip(Ws, bs, ys, Ns, ldc):
            want = P.dev_gemm_nt(fmt, xq, W, b, M, n, K).view(M, n)
            got = y.view(M, l)
            assert torch.equal(got[:, :n], want), (fmt, n)
            assert bool((got[:, n:] == 7.0).all()), "the padding of C stays untouched"
        ref = T.oracle_gemm_nt(fmt, xq.cpu().numpy(), Ws[2].cpu().numpy(), None, M, Ns[2], K)
        assert T.norm_err(ys[2].view(M, ldc[2])[:, :Ns[2]].cpu().numpy().reshape(-1), ref.reshape(-1)) <= TOL
    finally:
        L.ckq_set_gemm_policy(0)


def test_grouped_prefill_launch_two_wave_groups_and_fallback():
    """Q4_K, K = 2048: 168 tiles with eight K-steps take the two-wave-group form of the
    kernel (each single launch would be split along K instead, so the comparison is
    against the streaming kernel, token by token, at its tolerance); the same three
    matrices against 100 tokens are too few tiles for a group and are issued one by
    one, with the bits of the single calls."""
    import torch
    L = ckq.lib()
    K, Ns = 2048, [1536, 640, 392]
    Ws = [P.to_device(T.synth_weights("q4_k", n, K, seed=322 + i)) for i, n in enumerate(Ns)]
    for M in (500, 100):
        xq = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=321)), "q8_k", rows=M)
        ys = [torch.zeros(M * n, dtype=torch.float32, device="cuda") for n in Ns]
        L.ckq_set_gemm_policy(1)
        try:
            say("grouped prefill launch, K=2048", M)
            P.dev_matmul_sequence([("q4_k", xq, W, None, y, M, n, K) for W, y, n in zip(Ws, ys, Ns)])
            torch.cuda.synchronize()
            singles = [P.dev_gemm_nt("q4_k", xq, W, None, M, n, K).view(-1) for W, n in zip(Ws, Ns)]
            L.ckq_set_gemm_policy(2)
            streamed = [P.dev_gemm_nt("q4_k", xq, W, None, M, n, K).view(-1) for W, n in zip(Ws, Ns)]
        finally:
            L.ckq_set_gemm_policy(0)
        for y, one, st in zip(ys, singles, streamed):
            if M == 100:
                assert torch.equal(y, one)
            assert T.norm_err(y.cpu().numpy(), st.cpu().numpy()) <= 2e-6


# ---- host-pointer paths with the weight cache off, long contexts ---------------------------------------

def test_host_paths_with_weight_cache_off():
    """With uploads on every call (ckq_weights_set_cache(0)) each weight operand of
    a call has its own device buffer: the fused MLP (two weight matrices), a
    GEMV and an embedding lookup against the oracle."""
    L = ckq.lib()
    L.ckq_weights_clear()
    L.ckq_weights_set_cache(0)
    try:
        seq, E, I = 70, 256, 1024
        x = T.normal(seq * E, 0.0, 1.0, 61)
        W1 = T.synth_weights("q8_0", 2 * I, E, seed=62, std=0.25)
        W2 = T.synth_weights("q4_k", E, I, seed=63)
        say("fused MLP, cache off")
        got = P.fused_mlp_swiglu_prefill_w1w2_quant(x, W1, None, "q8_0", W2, None, "q4_k", seq, E, E, I, I)
        want = T.oracle_fused_mlp(x, W1, None, W2, None, "q4_k", seq, E, E, I, I)
        assert np.mean(np.abs(got - want) <= 1e-4 * np.abs(want).max()) >= 0.98
        assert np.abs(got - want).max() <= 5e-3 * np.abs(want).max()
        Wg = T.synth_weights("q4_k", 300, 1024, seed=64)
        xq = T.oracle_quantize(T.normal(1024, 0.0, 1.0, 65), "q8_k")
        say("GEMV, cache off")
        for _ in range(2):
            assert T.norm_err(P.gemv("q4_k", Wg, xq, 300, 1024), T.oracle_gemv("q4_k", Wg, xq, 300, 1024)) <= TOL
        vocab, D = 50, 256
        table = T.synth_weights("q8_0", vocab, D, seed=66)
        ids = np.array([3, 49, 0, 7], np.int32)
        say("embedding, cache off")
        out = P.embedding_forward("q8_0", ids, 4, vocab, table, None, D, D, 6, 0, fill=9.0)
        ref = T.np_dequant("q8_0", table).reshape(vocab, D)[ids].astype(np.float32)
        assert np.array_equal(out[:4], ref) and not out[4:].any()
        assert L.ckq_weights_resident(None) == 0
    finally:
        L.ckq_weights_set_cache(1)


def test_weight_cache_eviction_under_a_small_limit():
    """A bound on resident weights smaller than W1 + W2 of a fused MLP: the
    lookup of W2 must not drop W1, which the same call still holds (it is
    served uncached instead), alternating GEMVs evict each other, results stay
    those of the oracle and the resident bytes stay within the bound."""
    L = ckq.lib()
    L.ckq_weights_clear()
    seq, E, I = 70, 256, 1024
    x = T.normal(seq * E, 0.0, 1.0, 71)
    W1 = T.synth_weights("q8_0", 2 * I, E, seed=72, std=0.25)       # 557 056 bytes
    W2 = T.synth_weights("q4_k", E, I, seed=73)                     # 147 456 bytes
    Wa = T.synth_weights("q4_k", 600, 1024, seed=74)                # 345 600 bytes
    Wb = T.synth_weights("q6_k", 500, 1024, seed=75)                # 420 000 bytes
    xq = T.oracle_quantize(T.normal(1024, 0.0, 1.0, 76), "q8_k")
    limit = 600 * 1024
    assert W1.nbytes < limit < W1.nbytes + W2.nbytes and Wa.nbytes + Wb.nbytes > limit
    L.ckq_weights_set_limit(limit)
    try:
        want = T.oracle_fused_mlp(x, W1, None, W2, None, "q4_k", seq, E, E, I, I)
        for rep in range(2):
            say("fused MLP under a cache limit, call", rep)
            got = P.fused_mlp_swiglu_prefill_w1w2_quant(x, W1, None, "q8_0", W2, None, "q4_k", seq, E, E, I, I)
            assert np.mean(np.abs(got - want) <= 1e-4 * np.abs(want).max()) >= 0.98
            assert np.abs(got - want).max() <= 5e-3 * np.abs(want).max()
            nbytes = ctypes.c_size_t(0)
            L.ckq_weights_resident(ctypes.byref(nbytes))
            assert nbytes.value <= limit
        ya, yb = T.oracle_gemv("q4_k", Wa, xq, 600, 1024), T.oracle_gemv("q6_k", Wb, xq, 500, 1024)
        for rep in range(3):
            say("alternating GEMVs under a cache limit, round", rep)
            assert T.norm_err(P.gemv("q4_k", Wa, xq, 600, 1024), ya) <= TOL
            assert T.norm_err(P.gemv("q6_k", Wb, xq, 500, 1024), yb) <= TOL
            nbytes = ctypes.c_size_t(0)
            n = L.ckq_weights_resident(ctypes.byref(nbytes))
            assert n >= 1 and nbytes.value <= limit
    finally:
        L.ckq_weights_set_limit(0)
        L.ckq_weights_clear()


def test_embedding_context_window_beyond_grid_y():
    """context_window = 70 000 output rows (the reference zero-fills rows from
    token_count on): more rows than gridDim.y can index."""
    vocab, D, ctx, tokens = 64, 256, 70000, 5
    table = T.synth_weights("q4_k", vocab, D, seed=71)
    ids = np.array([1, 63, 0, 17, 5], np.int32)
    say("embedding with 70 000 context rows")
    out = P.embedding_forward("q4_k", ids, tokens, vocab, table, None, D, D, ctx, 0, fill=3.0)
    ref = T.np_dequant("q4_k", table).reshape(vocab, D)[ids].astype(np.float32)
    assert np.array_equal(out[:tokens], ref)
    assert not out[tokens:].any()


def test_f32act_gemv_with_more_tokens_than_grid_y():
    """The fp32-activation kernels take one token per launch row; 70 000 tokens
    go out as two launches over consecutive token ranges."""
    fmt, N, K, M = "q8_0", 8, 64, 70000
    W = T.random_blocks(fmt, N * (K // 32), 81)
    A = T.normal(M * K, 0.0, 1.0, 82)
    say("fp32-activation GEMM with 70 000 tokens")
    got = P.dev_gemm_nt_f32act(fmt, P.to_device(A), P.to_device(W), None, M, N, K).cpu().numpy().reshape(M, N)
    want = T.oracle_gemm_nt_f32act(fmt, A, W, None, M, N, K)
    assert T.norm_err(got, want) <= TOL
    assert T.norm_err(got[65530:65540], want[65530:65540]) <= TOL


# ---- Q4_K x Q8_K on 96-token tiles -------------------------------------------------------------------

Q4K_T96_SHAPES = [
    # (M, N, K): one, two and three token groups in the last tile, ragged rows, one to six K-blocks (odd and even)
    (96, 128, 512), (97, 130, 1024), (150, 300, 256), (33, 256, 768), (64, 200, 1536), (200, 128, 512), (500, 260, 1280),
]


def test_q4k_96_token_tiles_integer_block_sums_bit_exact():
    """The 96-token kernel forced for every shape: I1 / I2 per (token, row, block) against brute
    force - the carried group of each block included, whose sums are stored one block late - and the
    fp32 result of the dump build, of the production build and of the 64-token kernel agree bit for bit
    (neither splits K nor puts two wave groups on a tile at these sizes)."""
    L, D = ckq.lib(), ckq.dump_lib()       # each library has its own switch
    try:
        D.ckq_set_prefill_variant(P.FMT["q4_k"], 96)
        for M, N, K in Q4K_T96_SHAPES:
            W, A = rand_case("q4_k", N, K, 5 * M + N + K, tokens=M)
            say("q4_k 96-token tiles", M, N, K)
            Ad, Wd = P.to_device(A), P.to_device(W)
            b = P.to_device(T.normal(N, 0.0, 1.0, seed=N))
            L.ckq_set_prefill_variant(P.FMT["q4_k"], 96)
            c, sums = P.dev_gemm_block_sums("q4_k", Ad, Wd, b, M, N, K)
            assert np.array_equal(sums.cpu().numpy().astype(np.int64), np_block_sums("q4_k", W, A, M, N, K)), (M, N, K)
            L.ckq_set_gemm_policy(1)
            prod96 = P.dev_gemm_nt("q4_k", Ad, Wd, b, M, N, K).cpu().numpy()
            L.ckq_set_prefill_variant(P.FMT["q4_k"], 64)
            prod64 = P.dev_gemm_nt("q4_k", Ad, Wd, b, M, N, K).cpu().numpy()
            L.ckq_set_gemm_policy(0)
            assert np.array_equal(c.cpu().numpy(), prod96), (M, N, K)
            assert np.array_equal(prod96, prod64), (M, N, K)
            assert T.norm_err(prod96, T.oracle_gemm_nt("q4_k", A, W, b.cpu().numpy(), M, N, K)) <= TOL
    finally:
        L.ckq_set_gemm_policy(0)
        L.ckq_set_prefill_variant(P.FMT["q4_k"], 0)
        D.ckq_set_prefill_variant(P.FMT["q4_k"], 0)


def test_q4k_96_token_tiles_chosen_by_shape_and_grouped():
    """768 tokens x 8192 rows is one round of whole 96-token tiles: the default choice takes that kernel
    (same bits as the 64-token kernel forced, which does not split K here either).  Three ragged matrices
    against 500 tokens as ONE grouped launch of 96-token tiles: the bits of the single launches, the
    padding of C untouched."""
    import torch
    L = ckq.lib()
    try:
        M, N, K = 768, 8192, 512
        xq = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=401)), "q8_k", rows=M)
        W = P.to_device(T.synth_weights("q4_k", N, K, seed=402))
        say("q4_k tile by shape", M, N, K)
        L.ckq_set_gemm_policy(1)
        auto = P.dev_gemm_nt("q4_k", xq, W, None, M, N, K).clone()
        L.ckq_set_prefill_variant(P.FMT["q4_k"], 64)
        t64 = P.dev_gemm_nt("q4_k", xq, W, None, M, N, K).clone()
        L.ckq_set_prefill_variant(P.FMT["q4_k"], 96)
        t96 = P.dev_gemm_nt("q4_k", xq, W, None, M, N, K).clone()
        assert torch.equal(auto, t64) and torch.equal(auto, t96)
        rows = [0, 95, 96, 767]
        ref = T.oracle_gemm_nt("q4_k", xq.view(M, -1)[rows].cpu().numpy().reshape(-1), W.cpu().numpy(), None, len(rows), N, K)
        assert T.norm_err(auto.view(M, N)[rows].cpu().numpy().reshape(-1), ref.reshape(-1)) <= TOL

        M, K, Ns = 500, 1024, [1536, 640, 392]
        xq = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=411)), "q8_k", rows=M)
        Ws = [P.to_device(T.synth_weights("q4_k", n, K, seed=412 + i)) for i, n in enumerate(Ns)]
        bs = [None, P.to_device(T.normal(Ns[1], 0.0, 1.0, seed=420)), None]
        ldc = [n + 8 for n in Ns]
        ys = [torch.full((M * l,), 7.0, dtype=torch.float32, device="cuda") for l in ldc]
        say("q4_k grouped launch of 96-token tiles", M, Ns, K)
        P.dev_matmul_sequence([("q4_k", xq, W, b, y, M, n, K, l) for W, b, y, n, l in zip(Ws, bs, ys, Ns, ldc)])
        torch.cuda.synchronize()
        L.ckq_set_prefill_variant(P.FMT["q4_k"], 64)
        for W, b, y, n, l in zip(Ws, bs, ys, Ns, ldc):
            want = P.dev_gemm_nt("q4_k", xq, W, b, M, n, K).view(M, n)
            got = y.view(M, l)
            assert torch.equal(got[:, :n], want), n
            assert bool((got[:, n:] == 7.0).all()), "the padding of C stays untouched"
    finally:
        L.ckq_set_gemm_policy(0)
        L.ckq_set_prefill_variant(P.FMT["q4_k"], 0)


# ---- Q6_K x Q8_K, two blocks per CU -------------------------------------------------------------------

def test_q6k_paired_kernel_integer_block_sums_bit_exact_and_chosen_by_shape():
    """The paired 64-token Q6_K kernel (one LDS image of the weights, two blocks per CU) forced over ragged
    shapes and one to six K-blocks: the block sums against brute force, the fp32 result equal to the
    one-block-per-CU kernels' bit for bit.  512 tokens x 11008 rows leave the 128-token grid a third of a
    second round: the default choice takes the paired kernel there, with the same bits again."""
    import torch
    L, D = ckq.lib(), ckq.dump_lib()       # each library has its own switch
    q6 = P.FMT["q6_k"]
    try:
        for M, N, K in [(70, 200, 1024), (130, 384, 768), (33, 128, 256), (500, 260, 1536), (64, 130, 512)]:
            W, A = rand_case("q6_k", N, K, 7 * M + N + K, tokens=M)
            say("q6_k paired kernel", M, N, K)
            Ad, Wd = P.to_device(A), P.to_device(W)
            b = P.to_device(T.normal(N, 0.0, 1.0, seed=N))
            D.ckq_set_prefill_variant(q6, 2)
            c, sums = P.dev_gemm_block_sums("q6_k", Ad, Wd, b, M, N, K)
            assert np.array_equal(sums.cpu().numpy().astype(np.int64), np_block_sums("q6_k", W, A, M, N, K)), (M, N, K)
            L.ckq_set_gemm_policy(1)
            L.ckq_set_prefill_variant(q6, 2)
            pair = P.dev_gemm_nt("q6_k", Ad, Wd, b, M, N, K).cpu().numpy()
            L.ckq_set_prefill_variant(q6, 1)
            lone = P.dev_gemm_nt("q6_k", Ad, Wd, b, M, N, K).cpu().numpy()
            L.ckq_set_gemm_policy(0)
            assert np.array_equal(c.cpu().numpy(), pair), (M, N, K)
            assert np.array_equal(pair, lone), (M, N, K)
            assert T.norm_err(pair, T.oracle_gemm_nt("q6_k", A, W, b.cpu().numpy(), M, N, K)) <= TOL
        M, N, K = 512, 11008, 512
        xq = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=501)), "q8_k", rows=M)
        W = P.to_device(T.synth_weights("q6_k", N, K, seed=502))
        say("q6_k kernel by shape", M, N, K)
        L.ckq_set_gemm_policy(1)
        L.ckq_set_prefill_variant(q6, 0)
        auto = P.dev_gemm_nt("q6_k", xq, W, None, M, N, K).clone()
        L.ckq_set_prefill_variant(q6, 1)
        lone = P.dev_gemm_nt("q6_k", xq, W, None, M, N, K).clone()
        L.ckq_set_prefill_variant(q6, 2)
        pair = P.dev_gemm_nt("q6_k", xq, W, None, M, N, K).clone()
        assert torch.equal(auto, lone) and torch.equal(auto, pair)
    finally:
        L.ckq_set_gemm_policy(0)
        L.ckq_set_prefill_variant(q6, 0)
        D.ckq_set_prefill_variant(q6, 0)


def test_q5k_paired_kernel_integer_block_sums_bit_exact_and_chosen_by_tile_count():
    """The paired Q5_K kernel (one LDS image of the weights, two blocks per CU) forced over ragged shapes and
    one to six K-blocks: I1 / I2 against brute force, the fp32 result equal to the three-stage kernel's bit
    for bit.  640 tokens x 4096 rows are 320 tiles, more than CUs: the default choice takes the paired
    kernel, with the same bits again; three ragged matrices as one grouped launch of it likewise."""
    import torch
    L, D = ckq.lib(), ckq.dump_lib()       # each library has its own switch
    q5 = P.FMT["q5_k"]
    try:
        for M, N, K in [(70, 200, 1024), (130, 384, 768), (33, 128, 256), (500, 260, 1536), (64, 130, 512)]:
            W, A = rand_case("q5_k", N, K, 9 * M + N + K, tokens=M)
            say("q5_k paired kernel", M, N, K)
            Ad, Wd = P.to_device(A), P.to_device(W)
            b = P.to_device(T.normal(N, 0.0, 1.0, seed=N))
            D.ckq_set_prefill_variant(q5, 2)
            c, sums = P.dev_gemm_block_sums("q5_k", Ad, Wd, b, M, N, K)
            assert np.array_equal(sums.cpu().numpy().astype(np.int64), np_block_sums("q5_k", W, A, M, N, K)), (M, N, K)
            L.ckq_set_gemm_policy(1)
            L.ckq_set_prefill_variant(q5, 2)
            pair = P.dev_gemm_nt("q5_k", Ad, Wd, b, M, N, K).cpu().numpy()
            L.ckq_set_prefill_variant(q5, 1)
            lone = P.dev_gemm_nt("q5_k", Ad, Wd, b, M, N, K).cpu().numpy()
            L.ckq_set_gemm_policy(0)
            assert np.array_equal(c.cpu().numpy(), pair), (M, N, K)
            assert np.array_equal(pair, lone), (M, N, K)
            assert T.norm_err(pair, T.oracle_gemm_nt("q5_k", A, W, b.cpu().numpy(), M, N, K)) <= TOL
        M, N, K = 640, 4096, 512
        xq = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=601)), "q8_k", rows=M)
        W = P.to_device(T.synth_weights("q5_k", N, K, seed=602))
        say("q5_k kernel by tile count", M, N, K)
        L.ckq_set_gemm_policy(1)
        L.ckq_set_prefill_variant(q5, 0)
        auto = P.dev_gemm_nt("q5_k", xq, W, None, M, N, K).clone()
        L.ckq_set_prefill_variant(q5, 1)
        lone = P.dev_gemm_nt("q5_k", xq, W, None, M, N, K).clone()
        assert torch.equal(auto, lone)
        Ns = [1536, 2048, 904]
        Ws = [P.to_device(T.synth_weights("q5_k", n, K, seed=612 + i)) for i, n in enumerate(Ns)]
        ys = [torch.zeros(M * n, dtype=torch.float32, device="cuda") for n in Ns]
        L.ckq_set_prefill_variant(q5, 0)
        say("q5_k grouped launch of the paired kernel", M, Ns, K)
        P.dev_matmul_sequence([("q5_k", xq, Wj, None, y, M, n, K) for Wj, y, n in zip(Ws, ys, Ns)])
        torch.cuda.synchronize()
        L.ckq_set_prefill_variant(q5, 1)
        for Wj, y, n in zip(Ws, ys, Ns):
            assert torch.equal(y.view(M, n), P.dev_gemm_nt("q5_k", xq, Wj, None, M, n, K).view(M, n)), n
    finally:
        L.ckq_set_gemm_policy(0)
        L.ckq_set_prefill_variant(q5, 0)
        D.ckq_set_prefill_variant(q5, 0)


def test_q4k_96_token_tiles_full_size_equal_64_token_tiles():
    """The prefill shape at 1 000 tokens (ten whole 96-token tiles and one of 40 tokens per 128 rows, 946
    blocks, sixteen K-blocks): the 96-token kernel, taken by the default choice here, gives the bits of the
    64-token kernel for every output, and four tokens - first, last of a whole tile, first and last of the
    remainder tile - agree with the oracle."""
    import torch
    L = ckq.lib()
    q4 = P.FMT["q4_k"]
    M, N, K = 1000, 11008, 4096
    try:
        xq = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=701)), "q8_k", rows=M)
        W = P.to_device(T.synth_weights("q4_k", N, K, seed=702))
        b = P.to_device(T.normal(N, 0.0, 1.0, seed=703))
        say("q4_k 96-token tiles, full size", M, N, K)
        L.ckq_set_gemm_policy(1)
        L.ckq_set_prefill_variant(q4, 0)
        auto = P.dev_gemm_nt("q4_k", xq, W, b, M, N, K).clone()
        L.ckq_set_prefill_variant(q4, 96)
        t96 = P.dev_gemm_nt("q4_k", xq, W, b, M, N, K).clone()
        L.ckq_set_prefill_variant(q4, 64)
        t64 = P.dev_gemm_nt("q4_k", xq, W, b, M, N, K).clone()
        assert torch.equal(t96, t64) and torch.equal(auto, t96)
        rows = [0, 95, 960, 999]
        ref = T.oracle_gemm_nt("q4_k", xq.view(M, -1)[rows].cpu().numpy().reshape(-1), W.cpu().numpy(), b.cpu().numpy(), len(rows), N, K)
        assert T.norm_err(t96.view(M, N)[rows].cpu().numpy().reshape(-1), ref.reshape(-1)) <= TOL
    finally:
        L.ckq_set_gemm_policy(0)
        L.ckq_set_prefill_variant(q4, 0)
