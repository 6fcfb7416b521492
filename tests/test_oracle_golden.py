"""Pins the CPU oracle: golden vectors written from the compiled reference C
(tests/golden/make_golden.py), hand-computed known answers, closed forms and
brute force.  Runs on CPU."""
import ctypes
import os

import numpy as np
import pytest

import ckq_testlib as T
from ckq_testlib import ptr

FLOAT_TOL = 2e-6  # normalised; fp32 summation order differs at the ulp level between builds


# ---- fp16 -------------------------------------------------------------------

def test_fp16_to_fp32_exhaustive():
    O = T.oracle()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([O.orc_fp16_to_fp32(int(h)) for h in allh], dtype=np.float32)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all()


def test_fp32_to_fp16_rne():
    O = T.oracle()
    rng = np.random.default_rng(5)
    xs = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s
                         for s in (1e-8, 1e-7, 1e-5, 1e-3, 1.0, 100.0, 3e4, 7e4)])
    # exact ties between neighbouring halves, subnormal boundary, overflow edge
    xs = np.concatenate([xs, np.array([1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, 2 ** -24, 2 ** -25, 3 * 2 ** -25,
                                       65504.0, 65519.0, 65520.0, 6.1e-5, 0.0, -0.0], np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([O.orc_fp32_to_fp16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---- 6-bit scale unpack -----------------------------------------------------

# the five byte patterns of the reference's unittest/test_dequant_vs_llamacpp.c:293-300
# with scales/mins worked out by hand from the GGUF get_scale_min_k4 rule
SCALE_KAT = [
    ([236, 243, 254, 184, 172, 230, 235, 185, 123, 7, 255, 201],
     [44, 51, 62, 56, 59, 55, 63, 41], [44, 38, 43, 57, 39, 48, 63, 44]),
    ([0] * 12, [0] * 8, [0] * 8),
    ([255] * 12, [63] * 8, [63] * 8),
    ([0xC0] * 8 + [0] * 4, [0, 0, 0, 0, 48, 48, 48, 48], [0, 0, 0, 0, 48, 48, 48, 48]),
    ([0x3F] * 8 + [0xFF] * 4, [63, 63, 63, 63, 15, 15, 15, 15], [63, 63, 63, 63, 15, 15, 15, 15]),
]


@pytest.mark.parametrize("packed,sc_want,m_want", SCALE_KAT)
def test_scale_unpack_known_answers(packed, sc_want, m_want):
    O = T.oracle()
    s = np.array(packed, np.uint8)
    for fn in (O.orc_unpack_scales_k4, O.orc_unpack_scales_k4_kmask):
        sc = np.zeros(8, np.uint8)
        m = np.zeros(8, np.uint8)
        fn(ptr(s), ptr(sc), ptr(m))
        assert sc.tolist() == sc_want and m.tolist() == m_want


def test_scale_unpack_byte_and_word_forms_agree():
    O = T.oracle()
    rng = np.random.default_rng(11)
    for _ in range(2000):
        s = rng.integers(0, 256, 12, dtype=np.uint8)
        a, b, c, d = (np.zeros(8, np.uint8) for _ in range(4))
        O.orc_unpack_scales_k4(ptr(s), ptr(a), ptr(b))
        O.orc_unpack_scales_k4_kmask(ptr(s), ptr(c), ptr(d))
        assert np.array_equal(a, c) and np.array_equal(b, d)


# ---- dequantizers -------------------------------------------------------------

def test_q4_k_closed_form_block():
    """d=1.0, dmin=0.5, scales 2, mins 1 (sub-blocks 0-3) / 2 (4-7), every byte
    0x84: the block of the reference's test_dequant_vs_llamacpp.c:331-375."""
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([0x3C00], np.uint16).view(np.uint8)
    blk[2:4] = np.array([0x3800], np.uint16).view(np.uint8)
    blk[4:8] = 2
    blk[8:12] = 1
    blk[12:16] = 0x22
    blk[16:] = 0x84
    out = np.zeros(256, np.float32)
    T.oracle().orc_dequant_q4_k_row(ptr(blk), ptr(out), ctypes.c_size_t(256))
    want = np.zeros(256, np.float32)
    for g in range(4):
        lo, hi = (7.5, 15.5) if g < 2 else (7.0, 15.0)
        want[64 * g:64 * g + 32] = lo
        want[64 * g + 32:64 * g + 64] = hi
    assert np.array_equal(out, want)


@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q8_0"])
def test_dequant_matches_reference_golden(fmt):
    G = T.golden()
    w = G["deq_%s_w" % fmt]
    want = G["deq_%s_out" % fmt]
    out = np.zeros_like(want)
    getattr(T.oracle(), "orc_dequant_%s_row" % fmt)(ptr(w), ptr(out), ctypes.c_size_t(len(want)))
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    # the NumPy decoders used by the brute-force checks read the same layout
    assert np.allclose(T.np_dequant(fmt, w), want.astype(np.float64), rtol=1e-6, atol=1e-9)


def test_q5_k_fifth_bit_plane():
    """One block with a single set bit in qh: exactly one element gains 16."""
    for g in range(4):
        for half in range(2):
            for l in (0, 13, 31):
                blk = np.zeros(176, np.uint8)
                blk[0:2] = np.array([0x3C00], np.uint16).view(np.uint8)  # d = 1
                blk[4:8] = 1
                blk[12:16] = 0x01  # scales 4..7 = 1, mins 0
                blk[16 + l] = 1 << (2 * g + half)
                out = np.zeros(256, np.float32)
                T.oracle().orc_dequant_q5_k_row(ptr(blk), ptr(out), ctypes.c_size_t(256))
                want = np.zeros(256, np.float32)
                want[64 * g + 32 * half + l] = 16.0
                assert np.array_equal(out, want), (g, half, l)
                assert np.array_equal(T.np_dequant("q5_k", blk).astype(np.float32), want)


# ---- activation quantizers (bit-exact) -----------------------------------------

def test_quantize_q8_k_bit_exact_vs_reference():
    G = T.golden()
    x, want = G["q8k_in"], G["q8k_out"]
    got = T.oracle_quantize(x, "q8_k")
    assert np.array_equal(got, want)


def test_quantize_q8_k_invariants():
    x = T.normal(64 * 256, 0.0, 2.0, seed=77)
    b = T.np_decode_q8_k(T.oracle_quantize(x, "q8_k"))
    q = b["q"]
    assert np.array_equal(q.reshape(-1, 16, 16).sum(axis=2), b["bsums"])
    xb = x.reshape(-1, 256)
    arg = np.argmax(np.abs(xb), axis=1)
    assert np.all(q[np.arange(len(arg)), arg] == -127)
    assert np.allclose(b["d"] * -127.0, xb[np.arange(len(arg)), arg], rtol=1e-6)
    # round trip within half a step
    assert np.max(np.abs(b["d"][:, None] * q - xb) / np.abs(b["d"][:, None])) <= 0.5 + 1e-3


def test_quantize_batch_equals_row_loop():
    x = T.normal(5 * 768, seed=9)
    whole = T.oracle_quantize(x, "q8_k", rows=5)
    rows = np.concatenate([T.oracle_quantize(x[r * 768:(r + 1) * 768], "q8_k") for r in range(5)])
    assert np.array_equal(whole, rows)
    whole = T.oracle_quantize(x, "q8_0", rows=5)
    rows = np.concatenate([T.oracle_quantize(x[r * 768:(r + 1) * 768], "q8_0") for r in range(5)])
    assert np.array_equal(whole, rows)


def test_quantize_q8_0_bit_exact_vs_reference():
    G = T.golden()
    got = T.oracle_quantize(G["q80_in"], "q8_0")
    assert np.array_equal(got, G["q80_out"])


# ---- integer sub-block dots ------------------------------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_subdots_brute_force(fmt, kind):
    G = T.golden()
    M, K, _ = (int(v) for v in G["shape"])
    W = G["w_%s_%s" % (fmt, kind)]
    xq = G["act_q80" if fmt == "q8_0" else "act_q8k"][:T.row_bytes(T.act_fmt(fmt), K)].copy()
    assert np.array_equal(T.oracle_subdots(fmt, W, xq, M, K), T.np_subdots(fmt, W, xq, M, K))


# ---- GEMV / GEMM against the reference builds ------------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("kind", ["rand", "enc"])
@pytest.mark.parametrize("build", ["avx2", "avx512"])
def test_gemv_matches_reference(fmt, kind, build):
    G = T.golden()
    M, K, _ = (int(v) for v in G["shape"])
    W = G["w_%s_%s" % (fmt, kind)]
    xq = G["act_q80" if fmt == "q8_0" else "act_q8k"]
    y = T.oracle_gemv(fmt, W, xq, M, K)
    assert T.norm_err(y, G["y_%s_%s_%s" % (fmt, kind, build)]) <= FLOAT_TOL


@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_gemm_nt_with_bias_matches_reference(fmt, kind):
    G = T.golden()
    N, K, M = (int(v) for v in G["shape"])
    W = G["w_%s_%s" % (fmt, kind)]
    A = G["act_q80" if fmt == "q8_0" else "act_q8k"]
    c = T.oracle_gemm_nt(fmt, A, W, G["bias"], M, N, K)
    assert T.norm_err(c, G["c_%s_%s_avx2" % (fmt, kind)]) <= FLOAT_TOL
    # token 0 without bias is the GEMV
    c0 = T.oracle_gemm_nt(fmt, A, W, None, 1, N, K)
    y = T.oracle_gemv(fmt, W, A, N, K)
    assert T.norm_err(c0, y) <= FLOAT_TOL


@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_variants_match_reference(kind):
    G = T.golden()
    M, K, TOK = (int(v) for v in G["shape"])
    O = T.oracle()
    xq, xf = G["act_q8k"], G["act_f32"]
    # Q4_K scalar reference, and stored-bsums semantics (zeroed bsums)
    W = G["w_q4_k_" + kind]
    assert T.norm_err(T.oracle_gemv("q4_k", W, xq, M, K), G["y_q4_k_%s_ref" % kind]) <= FLOAT_TOL
    y = T.oracle_gemv("q4_k", W, G["act_q8k_zero_bsums"], M, K)
    assert T.norm_err(y, G["y_q4_k_%s_zero_bsums" % kind]) <= FLOAT_TOL
    assert T.norm_err(y, G["y_q4_k_%s_avx2" % kind]) > 1e-3  # the min term really is gone
    # row-split union equals serial
    yp = np.zeros(M, np.float32)
    for ith in range(5):
        O.orc_gemv_q4_k_q8_k_parallel(ptr(yp), ptr(W), ptr(xq), M, K, ith, 5)
    assert np.array_equal(yp, T.oracle_gemv("q4_k", W, xq, M, K))
    assert T.norm_err(yp, G["y_q4_k_%s_parallel5" % kind]) <= FLOAT_TOL
    # Q5_K: zero bsums, fp32 adapter
    W = G["w_q5_k_" + kind]
    y = T.oracle_gemv("q5_k", W, G["act_q8k_zero_bsums"], M, K)
    assert T.norm_err(y, G["y_q5_k_%s_zero_bsums" % kind]) <= FLOAT_TOL
    y = np.zeros(M, np.float32)
    O.orc_gemv_q5_k(ptr(y), ptr(W), ptr(xf), M, K)
    assert T.norm_err(y, G["y_q5_k_%s_f32act" % kind]) <= FLOAT_TOL
    c = np.zeros(TOK * M, np.float32)
    O.orc_gemm_nt_q5_k(ptr(xf), ptr(W), ptr(G["bias"]), ptr(c), TOK, M, K)
    assert T.norm_err(c, G["c_q5_k_%s_f32act" % kind]) <= FLOAT_TOL
    # Q6_K: element-wise scalar form, bsums are not read, vec_dot
    W = G["w_q6_k_" + kind]
    assert T.norm_err(T.oracle_gemv("q6_k", W, xq, M, K, "orc_gemv_q6_k_q8_k_ref"),
                      G["y_q6_k_%s_ref" % kind]) <= 1e-5
    y = T.oracle_gemv("q6_k", W, G["act_q8k_zero_bsums"], M, K)
    assert np.array_equal(y, T.oracle_gemv("q6_k", W, xq, M, K))
    assert T.norm_err(y, G["y_q6_k_%s_zero_bsums" % kind]) <= FLOAT_TOL
    s = np.zeros(1, np.float32)
    O.orc_vec_dot_q6_k_q8_k(K, ptr(s), ptr(W), ptr(xq))
    assert T.norm_err(s, G["s_q6_k_%s_vecdot" % kind]) <= FLOAT_TOL
    # Q8_0: fp32 activations, vec_dot, AVX2 lane order
    W = G["w_q8_0_" + kind]
    y = np.zeros(M, np.float32)
    O.orc_gemv_q8_0(ptr(y), ptr(W), ptr(xf), M, K)
    assert T.norm_err(y, G["y_q8_0_%s_f32act" % kind]) <= 1e-5
    s = np.zeros(1, np.float32)
    O.orc_vec_dot_q8_0_q8_0(K, ptr(s), ptr(W), ptr(G["act_q80"]))
    assert T.norm_err(s, G["s_q8_0_%s_vecdot" % kind]) <= FLOAT_TOL


@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_lane_order_variants_bit_identical_to_avx2_build(kind):
    """The 8-lane restatements follow the AVX2 routines' summation order
    exactly, so they reproduce that build's fp32 results bit for bit."""
    G = T.golden()
    M, K, _ = (int(v) for v in G["shape"])
    y = T.oracle_gemv("q6_k", G["w_q6_k_" + kind], G["act_q8k"], M, K)
    assert np.array_equal(y.view(np.uint32), G["y_q6_k_%s_avx2" % kind].view(np.uint32))
    y = T.oracle_gemv("q8_0", G["w_q8_0_" + kind], G["act_q80"], M, K, "orc_gemv_q8_0_q8_0_lanes8")
    assert np.array_equal(y.view(np.uint32), G["y_q8_0_%s_avx2" % kind].view(np.uint32))

# ---- fp32 activations, no activation quantization ----------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_fp32_activation_kernels_match_reference(fmt, kind):
    """gemv_q4_k / gemv_q6_k / gemm_nt_q4_k / gemm_nt_q6_k / gemm_nt_q8_0: the
    weights are dequantized on the fly and dotted with fp32 activations.  Golden
    outputs come from both reference builds (AVX2 and AVX-512 sum in different
    orders); the closed form is dequantize-then-matmul in fp64."""
    G = T.golden()
    M, K, TOK = (int(v) for v in G["shape"])
    O = T.oracle()
    W, xf, bias = G["w_%s_%s" % (fmt, kind)], G["act_f32"], G["bias"]
    want = T.np_dequant(fmt, W).reshape(M, K).astype(np.float64) @ xf.reshape(TOK, K).T.astype(np.float64)   # [M, TOK]
    if fmt != "q8_0":
        y = np.zeros(M, np.float32)
        getattr(O, "orc_gemv_" + fmt)(ptr(y), ptr(W), ptr(xf), M, K)
        for build in ("avx2", "avx512"):
            assert T.norm_err(y, G["y_%s_%s_f32w_%s" % (fmt, kind, build)]) <= 1e-5
        assert T.norm_err(y, want[:, 0]) <= 1e-5
        # gemm_q*_k layout: Y[n*M + row]
        Y = np.zeros(TOK * M, np.float32)
        getattr(O, "orc_gemm_" + fmt)(ptr(Y), ptr(W), ptr(xf), M, TOK, K)
        assert T.norm_err(Y.reshape(TOK, M), want.T) <= 1e-5
    c = np.zeros(TOK * M, np.float32)
    getattr(O, "orc_gemm_nt_" + fmt)(ptr(xf), ptr(W), ptr(bias), ptr(c), TOK, M, K)
    for build in ("avx2", "avx512"):
        assert T.norm_err(c, G["c_%s_%s_f32w_%s" % (fmt, kind, build)]) <= 1e-5
    assert T.norm_err(c.reshape(TOK, M), want.T + bias[None, :]) <= 1e-5
    # a dropped min term, a wrong nibble order or a missing -32 would be far outside this
    c0 = np.zeros(TOK * M, np.float32)
    getattr(O, "orc_gemm_nt_" + fmt)(ptr(xf), ptr(W), None, ptr(c0), TOK, M, K)
    assert np.allclose(c - c0, np.tile(bias, TOK), atol=1e-5 * max(1.0, np.abs(c).max()))

# ---- fused producer: rmsnorm -> Q8_K ---------------------------------------------------

def test_rmsnorm_q8_k_fused_bit_exact_vs_reference():
    """Both reference builds produce the same bytes; the oracle reproduces them
    (sum of squares as fused multiply-adds in eight strided lanes).  The variant
    that rounds the product before the add is a different function: it must
    differ somewhere on enough data, which pins the choice."""
    G = T.golden()
    O = T.oracle()
    TF, DF, AF = (int(v) for v in G["rms_shape"])
    x, g, eps = G["rms_in"], G["rms_gamma"], float(G["rms_eps"][0])
    out = np.zeros_like(G["rms_out"])
    O.orc_rmsnorm_q8_k_fused(ptr(x), ptr(g), ptr(out), TF, DF, AF, ctypes.c_float(eps))
    assert np.array_equal(out, G["rms_out"])
    blocks = out.reshape(-1, 292)
    # the zeroed input block gives an all-zero output block
    assert not blocks[1 * (DF // 256) + 1].any()
    # scale from the largest magnitude: d is negative, and some quant is exactly +-127
    d = blocks[:, :4].copy().view(np.float32).reshape(-1)
    qs = blocks[:, 4:260].view(np.int8)
    live = d != 0
    assert np.all(d[live] < 0) and np.all(np.abs(qs[live]).max(axis=1) == 127)
    # bsums are the sums of 16
    bs = blocks[:, 260:].copy().view(np.int16)
    assert np.array_equal(bs, qs.reshape(-1, 16, 16).sum(axis=2).astype(np.int16))
    # closed form: dequantized output is rmsnorm(x)*gamma within half a quantization step
    xm = x.reshape(TF, AF)[:, :DF].astype(np.float64)
    want = xm / np.sqrt((xm ** 2).mean(axis=1, keepdims=True) + eps) * g.astype(np.float64)
    got = (qs.astype(np.float64) * d[:, None].astype(np.float64)).reshape(TF, DF)
    step = np.abs(d).reshape(TF, DF // 256).repeat(256, axis=1)
    assert np.all(np.abs(got - want) <= 0.5001 * step + 1e-6 * np.abs(want))


def test_rmsnorm_q8_k_fused_fma_choice_is_pinned():
    O = T.oracle()
    TF, DF = 64, 1024
    x = T.normal(TF * DF, 0.0, 30.0, seed=77)
    g = T.normal(DF, 1.0, 0.3, seed=78)
    a = np.zeros(TF * (DF // 256) * 292, np.uint8)
    b = np.zeros_like(a)
    O.orc_rmsnorm_q8_k_fused(ptr(x), ptr(g), ptr(a), TF, DF, DF, ctypes.c_float(1e-6))
    O.orc_rmsnorm_q8_k_fused_nofma(ptr(x), ptr(g), ptr(b), TF, DF, DF, ctypes.c_float(1e-6))
    assert (a != b).sum() > 0          # the two restatements are distinguishable ...
    assert (a != b).sum() < a.size // 100   # ... and differ only by rounding flips

# ---- quantized embedding lookup ----------------------------------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("add_pos", [0, 1])
def test_embedding_forward_bit_exact_vs_reference(fmt, add_pos):
    G = T.golden()
    VOC, ED, AED, CTX, NTOK = (int(v) for v in G["emb_shape"])
    ids, pos, tab = G["emb_ids"], G["emb_pos"], G["emb_table_" + fmt]
    out = np.full(CTX * AED, 9.0, np.float32)
    T.oracle().orc_embedding_forward(T.FMT[fmt], ptr(ids), NTOK, VOC, ptr(tab), ptr(pos), ptr(out), ED, AED, CTX, add_pos)
    want = G["emb_out_%s_pos%d" % (fmt, add_pos)]
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    # what the lookup must mean, from the format decoders: gathered rows, clamped ids, padding
    o = out.reshape(CTX, AED)
    rows = T.np_dequant(fmt, tab).reshape(VOC, AED)
    p = pos.reshape(CTX, AED)
    for t in range(NTOK):
        idx = int(ids[t]) if 0 <= ids[t] < VOC else 0
        exp = rows[idx, :ED] + (p[t, :ED] if add_pos else 0.0)
        assert np.allclose(o[t, :ED], exp, rtol=1e-6, atol=1e-7)
        assert np.all(o[t, ED:] == 0.0)
    assert np.all(o[NTOK:] == 0.0)


# ---- Q5_0 weights x Q8_0 activations ------------------------------------------------------------

@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_q5_0_q8_0_vs_reference(kind):
    """gemv / gemm_nt / vec_dot of both reference builds within the summation-order
    tolerance; the scalar _ref routine (the order restated here) bit for bit; the
    integer block dots against a NumPy decoder written from the format definition;
    and the Q5_0 -> Q8_0 block conversion, under which every dot is unchanged."""
    G = T.golden()
    O = T.oracle()
    ROWS, K, TOK = (int(v) for v in G["shape"])
    W, xq, bias = G["w_q5_0_" + kind], G["act_q80"], G["bias"]
    y = T.oracle_gemv("q5_0", W, xq, ROWS, K)
    c = T.oracle_gemm_nt("q5_0", xq, W, bias, TOK, ROWS, K)
    for tag in ("avx2", "avx512"):
        assert T.norm_err(y, G["y_q5_0_%s_%s" % (kind, tag)]) <= 2e-6
        assert T.norm_err(c, G["c_q5_0_%s_%s" % (kind, tag)].reshape(TOK, ROWS)) <= 2e-6
    s = np.zeros(1, np.float32)
    O.orc_vec_dot_q5_0_q8_0(K, ptr(s), ptr(W), ptr(xq))
    assert s.view(np.uint32)[0] == G["s_q5_0_%s_vecdot_ref" % kind].view(np.uint32)[0]
    assert abs(float(s[0]) - float(G["s_q5_0_%s_vecdot" % kind][0])) <= 2e-6 * np.abs(y).max()
    # integers, from the format definition
    x0 = xq[:T.row_bytes("q8_0", K)].copy()
    sub = T.oracle_subdots("q5_0", W, x0, ROWS, K)
    assert np.array_equal(sub, T.np_subdots("q5_0", W, x0, ROWS, K))
    # closed form of the row sums in float64
    wv = T.np_dequant("q5_0", W).reshape(ROWS, K)
    xv = T.np_dequant("q8_0", xq).reshape(TOK, K)
    assert np.allclose(y, wv @ xv[0], rtol=0, atol=2e-6 * np.abs(y).max())
    # conversion to Q8_0 blocks keeps every value and scale
    w8 = np.zeros(len(W) // 22 * 34, np.uint8)
    O.orc_q5_0_to_q8_0(ptr(W), ptr(w8), ctypes.c_size_t(len(W) // 22))
    assert np.array_equal(T.np_dequant("q8_0", w8), T.np_dequant("q5_0", W))
    assert np.array_equal(T.oracle_subdots("q8_0", w8, x0, ROWS, K), sub)
    assert T.norm_err(T.oracle_gemv("q8_0", w8, xq, ROWS, K), y) <= 2e-6


def test_fused_mlp_q5_0_gate_up_vs_reference():
    G = T.golden()
    SEQ, ED, AED, ID, AID = (int(v) for v in G["mlp_shape"])
    out = T.oracle_fused_mlp(G["mlp_x"], G["mlp_w1_q5_0"], G["mlp_b1"], G["mlp_w2_q4_k"], G["mlp_b2"], "q4_k",
                             SEQ, ED, AED, ID, AID, w1_fmt="q5_0")
    for tag in ("avx2", "avx512"):
        assert T.norm_err(out, G["mlp_out_q5_0w1_q4_k_%s" % tag].reshape(SEQ, AED)) <= 2e-6, tag


# ---- fused prefill MLP ----------------------------------------------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q6_k"])
def test_fused_mlp_swiglu_prefill_vs_reference(fmt):
    """The compiled reference (70 tokens: one full tile of 64 and a ragged one)
    against the restatement, and the restatement's stages against what they must
    mean: SiLU(gate)*up in float64, Q8_K of it, the down GEMM of that."""
    G = T.golden()
    SEQ, ED, AED, ID, AID = (int(v) for v in G["mlp_shape"])
    x, w1, b1, b2, w2 = G["mlp_x"], G["mlp_w1"], G["mlp_b1"], G["mlp_b2"], G["mlp_w2_" + fmt]
    out, gu, hq = T.oracle_fused_mlp(x, w1, b1, w2, b2, fmt, SEQ, ED, AED, ID, AID, want_intermediates=True)
    for tag in ("avx2", "avx512"):
        want = G["mlp_out_%s_%s" % (fmt, tag)].reshape(SEQ, AED)
        assert T.norm_err(out, want) <= 2e-6, tag
    # stage 1: gate and up are the Q8_0 GEMM of the quantized input (already pinned on its own)
    xq = T.oracle_quantize(x, "q8_0", rows=SEQ)
    c = T.oracle_gemm_nt("q8_0", xq, w1, b1, SEQ, 2 * AID, AED)
    up = gu[:, AID:]
    assert np.array_equal(up.view(np.uint32), c[:, AID:].view(np.uint32))
    # stage 2: the activation, against float64
    g64 = c[:, :AID].astype(np.float64)
    want_h = g64 / (1.0 + np.exp(-g64)) * up.astype(np.float64)
    assert np.all(np.abs(gu[:, :AID] - want_h) <= 4e-7 * np.abs(want_h) + 1e-30)
    # stage 3: Q8_K of exactly those floats
    assert np.array_equal(hq, T.oracle_quantize(np.ascontiguousarray(gu[:, :AID]).reshape(-1), "q8_k", rows=SEQ))
    # stage 4: the down GEMM of exactly those blocks
    assert np.array_equal(out.view(np.uint32), T.oracle_gemm_nt(fmt, hq, w2, b2, SEQ, AED, AID).view(np.uint32))


def test_fused_mlp_rejects_what_the_reference_rejects():
    G = T.golden()
    SEQ, ED, AED, ID, AID = (int(v) for v in G["mlp_shape"])
    O = T.oracle()
    x, w1, w2 = G["mlp_x"], G["mlp_w1"], G["mlp_w2_q4_k"]
    for bad in (dict(w1=T.CK_DT["q4_k"]), dict(w2=T.CK_DT["q8_0"]), dict(aed=AED + 8), dict(aid=AID + 32), dict(seq=0)):
        out = np.full(SEQ * AED, 7.0, np.float32)
        O.orc_fused_mlp_swiglu_prefill_w1w2_quant(ptr(x), ptr(w1), None, bad.get("w1", T.CK_DT["q8_0"]), ptr(w2), None,
                                                  bad.get("w2", T.CK_DT["q4_k"]), ptr(out), bad.get("seq", SEQ), ED,
                                                  bad.get("aed", AED), ID, bad.get("aid", AID), None, None)
        assert np.all(out == 7.0), bad


# ---- exact evaluation: dequantize-then-fp64 matmul ---------------------------------

@pytest.mark.parametrize("fmt", ["q4_k", "q5_k", "q6_k", "q8_0"])
@pytest.mark.parametrize("kind", ["rand", "enc"])
def test_exact_equals_dequant_matmul(fmt, kind):
    G = T.golden()
    M, K, _ = (int(v) for v in G["shape"])
    W = G["w_%s_%s" % (fmt, kind)]
    af = T.act_fmt(fmt)
    xq = G["act_q80" if fmt == "q8_0" else "act_q8k"][:T.row_bytes(af, K)].copy()
    want = T.np_dequant(fmt, W).reshape(M, K) @ T.np_dequant(af, xq)
    got = T.oracle_exact(fmt, W, xq, M, K)
    assert T.norm_err(got, want) <= 1e-12
    # and every fp32 kernel order approximates it
    assert T.norm_err(T.oracle_gemv(fmt, W, xq, M, K), want) <= 1e-5


def test_encoders_round_trip():
    """The weight encoders emit format-valid blocks: dequant(quant(w)) is
    within one quantisation step of w, and an all-zero row encodes to zeros."""
    S = T.synth()
    w = T.normal(16 * 256, 0.0, 0.02, seed=3)
    for fmt, steps in (("q4_k", 15), ("q5_k", 31), ("q6_k", 63), ("q8_0", 254)):
        out = np.zeros(T.row_bytes(fmt, len(w)), np.uint8)
        assert S.ckq_synth_quantize(T.FMT[fmt], ptr(w), ptr(out), ctypes.c_size_t(len(w))) == 0
        back = T.np_dequant(fmt, out)
        span = np.ptp(w.reshape(-1, T.ELEMS[fmt] if fmt == "q8_0" else 32), axis=1).max()
        assert np.max(np.abs(back - w)) <= 1.5 * span / steps
        z = np.zeros(256, np.float32)
        outz = np.zeros(T.row_bytes(fmt, 256), np.uint8)
        S.ckq_synth_quantize(T.FMT[fmt], ptr(z), ptr(outz), ctypes.c_size_t(256))
        assert np.all(T.np_dequant(fmt, outz) == 0.0)
    # non-zero dmin so the bsums half of the kernels is exercised
    out = np.zeros(T.row_bytes("q4_k", len(w)), np.uint8)
    S.ckq_synth_quantize(T.FMT["q4_k"], ptr(w), ptr(out), ctypes.c_size_t(len(w)))
    assert np.all(T.np_decode_q4_k(out)["dmin"] > 0)


def test_cpu_timing_harness_computes_what_it_times():
    """The CPU-baseline harness (persistent threads, one barrier-bracketed round
    per call) runs the split kernel it is handed: the output of its rounds is the
    serial GEMV's, every round is timed, bad arguments are refused."""
    import ctypes
    M, K, nth, iters = 203, 512, 3, 4
    W = T.synth_weights("q4_k", M, K, seed=77)
    xq = T.oracle_quantize(T.normal(K, seed=78), "q8_k")
    orc = T.oracle()
    orc.orc_time_split_gemv.restype = ctypes.c_int
    orc.orc_time_split_gemv.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.c_void_p]
    fn = ctypes.cast(orc.orc_gemv_q4_k_q8_k_parallel, ctypes.c_void_p)
    y = np.full(M, np.nan, np.float32)
    sec = np.zeros(iters, np.float64)
    assert orc.orc_time_split_gemv(fn, T.ptr(y), T.ptr(W), T.ptr(xq), M, K, nth, iters, T.ptr(sec)) == 0
    assert np.array_equal(y, T.oracle_gemv("q4_k", W, xq, M, K))
    assert np.all(sec > 0)
    assert orc.orc_time_split_gemv(fn, T.ptr(y), T.ptr(W), T.ptr(xq), M, K, 0, iters, T.ptr(sec)) == -1
    assert orc.orc_time_split_gemv(None, T.ptr(y), T.ptr(W), T.ptr(xq), M, K, nth, iters, T.ptr(sec)) == -1


def test_sanitizer_pass_over_cpu_code():
    """The oracle, the synthetic-data encoders and the library's HIP-free host
    helpers built with -fsanitize=address,undefined and driven over ragged
    shapes, extreme inputs and malformed manifest lines (oracle/asan_harness.c):
    no report, exit status 0."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(["make", "-C", os.path.join(root, "oracle"), "asan"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([os.path.join(root, "oracle", "asan_harness")], capture_output=True, text=True,
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", LD_PRELOAD=""))
    assert r.returncode == 0 and "ok" in r.stdout, (r.stdout + r.stderr)[-3000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr
