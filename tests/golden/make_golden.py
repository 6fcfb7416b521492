#!/usr/bin/env python3
"""Write the golden vectors for the quantized dequant-dot path.

The expected outputs come from the reference engine's own C kernels, compiled
from the reference checkout by `make -C oracle ref` into
oracle/_ref/libckref_avx2.so / libckref_avx512.so and called here through
ctypes (dispatch entry points: what a production x86 build runs).  No
reference Python is imported.  Inputs come from this repository's seeded
generator and are stored with the outputs, so the fixtures stand alone.

Build flags of the two reference builds are recorded in the fixture
(`flags_avx2`, `flags_avx512`).  fp32 kernel outputs of both builds are kept:
integers are pinned exactly, floats to tolerance.

Run from the repository root:  python tests/golden/make_golden.py
"""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), "..", ".."))
REFDIR = os.path.join(ROOT, "oracle", "_ref")
SYNTH = os.path.join(ROOT, "c-kernel-engine_amd", "csrc", "libckq_synth.so")
OUT = os.path.join(ROOT, "tests", "golden", "quant_path_golden.npz")

FMT = {"q4_k": 0, "q5_k": 1, "q6_k": 2, "q8_0": 3, "q8_k": 4, "q5_0": 5}
BLK = {"q4_k": 144, "q5_k": 176, "q6_k": 210, "q8_0": 34, "q8_k": 292, "q5_0": 22}
ELEMS = {"q4_k": 256, "q5_k": 256, "q6_k": 256, "q8_0": 32, "q8_k": 256, "q5_0": 32}

c_f32p = ctypes.POINTER(ctypes.c_float)
vp = ctypes.c_void_p


def ptr(a):
    return a.ctypes.data_as(vp)


def load():
    libs = {}
    for tag in ("avx2", "avx512"):
        path = os.path.join(REFDIR, "libckref_%s.so" % tag)
        if not os.path.exists(path):
            sys.exit("missing %s: run `make -C oracle ref` first" % path)
        libs[tag] = ctypes.CDLL(path)
    return libs, ctypes.CDLL(SYNTH)


def normal(S, n, mean, std, seed):
    out = np.empty(n, dtype=np.float32)
    S.ckq_synth_normal(ptr(out), ctypes.c_size_t(n), ctypes.c_float(mean), ctypes.c_float(std), ctypes.c_uint64(seed))
    return out


def synth_weights(S, fmt, rows, k, seed):
    out = np.zeros(rows * (k // ELEMS[fmt]) * BLK[fmt], dtype=np.uint8)
    rc = S.ckq_synth_weights(FMT[fmt], ptr(out), rows, k, ctypes.c_float(0.0), ctypes.c_float(0.02), ctypes.c_uint64(seed))
    assert rc == 0
    return out


def random_blocks(S, fmt, nblocks, seed):
    out = np.zeros(nblocks * BLK[fmt], dtype=np.uint8)
    rc = S.ckq_synth_random_blocks(FMT[fmt], ptr(out), ctypes.c_size_t(nblocks), ctypes.c_uint64(seed))
    assert rc == 0
    return out


def q8k_edge_inputs():
    """256-element rows that exercise the quantizer's special cases."""
    rows = []
    z = np.zeros(256, np.float32)
    rows.append(z.copy())                                   # all zero -> zero block
    a = z.copy(); a[7] = -3.0; a[200] = 3.0                 # tie: first (negative) wins
    rows.append(a)
    a = z.copy(); a[7] = 3.0; a[200] = -3.0                 # tie: first (positive) wins
    rows.append(a)
    a = z.copy(); a[0] = -127.0                             # iscale = 1: exact halves round to even
    a[1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    rows.append(a)
    a = z.copy(); a[0] = 127.0                              # iscale = -1
    a[1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    rows.append(a)
    rows.append(np.full(256, 1.0, np.float32))              # constant
    rows.append(np.full(256, -1e-30, np.float32))           # tiny normal
    rows.append(np.full(256, 1e-41, np.float32))            # fp32 subnormals
    a = (np.arange(256, dtype=np.float32) - 128.0) * 1e30   # huge
    rows.append(a)
    a = z.copy(); a[255] = 1e-3                             # single non-zero at the end
    rows.append(a)
    a = np.linspace(-1.0, 1.0, 256).astype(np.float32)      # both extremes equal magnitude
    rows.append(a)
    # magnitudes below 127/FLT_MAX: the inverse scale is infinite, products are +-inf
    # or NaN (0 * inf), and cvtps2dq turns all of them into INT_MIN -> -128
    a = (np.where(np.arange(256) % 3 == 0, -1.0, 1.0) * np.geomspace(1e-38, 1e-41, 256)).astype(np.float32)
    rows.append(a)                                          # mixed signs, 1e-38 .. 1e-41
    a = np.full(256, -2e-39, np.float32); a[100] = 1e-40    # a single +tiny among -tiny
    rows.append(a)
    a = z.copy(); a[3] = 3e-38; a[77] = -1e-39              # zeros beside an infinite inverse scale
    rows.append(a)
    return np.concatenate(rows)


def q80_edge_inputs():
    """32-element blocks whose inverse scale 127/amax overflows to +inf."""
    rows = []
    a = (np.where(np.arange(32) % 2 == 0, 1.0, -1.0) * np.geomspace(1e-38, 1e-41, 32)).astype(np.float32)
    rows.append(a)                                          # mixed signs
    a = np.full(32, -2e-39, np.float32); a[5] = 1e-40       # a single +tiny among -tiny
    rows.append(a)
    a = np.zeros(32, np.float32); a[9] = 2e-38              # zeros: 0 * inf = NaN
    rows.append(a)
    return np.concatenate(rows)


def main():
    libs, S = load()
    G = {}
    for tag in libs:
        with open(os.path.join(REFDIR, "flags_%s.txt" % tag)) as f:
            G["flags_" + tag] = np.array(f.read().strip())

    # ---- activation quantizers (bit-exact) --------------------------------
    x_k = np.concatenate([normal(S, 48 * 256, 0.0, 1.0, 101), q8k_edge_inputs(),
                          normal(S, 8 * 256, 0.0, 300.0, 102), normal(S, 8 * 256, 0.0, 1e-4, 103)])
    G["q8k_in"] = x_k
    outs = {}
    for tag, L in libs.items():
        o = np.zeros(len(x_k) // 256 * 292, np.uint8)
        L.quantize_row_q8_k(ptr(x_k), ptr(o), len(x_k))
        outs[tag] = o
    assert np.array_equal(outs["avx2"], outs["avx512"]), "q8_k quantizer differs between builds"
    G["q8k_out"] = outs["avx2"]
    # batch entry point == row loop
    o = np.zeros_like(outs["avx2"])
    libs["avx2"].quantize_batch_q8_k(ptr(x_k), ptr(o), len(x_k) // 768, 768)
    assert np.array_equal(o, outs["avx2"])

    x_0 = np.concatenate([normal(S, 96 * 32, 0.0, 1.0, 111), np.zeros(32, np.float32),
                          np.full(32, 2.5, np.float32), normal(S, 16 * 32, 0.0, 1e-6, 112),
                          normal(S, 16 * 32, 0.0, 1e4, 113),
                          (np.arange(32, dtype=np.float32) - 16.0) / 2.0 * (127.0 / 127.0),
                          q80_edge_inputs()])
    G["q80_in"] = x_0
    outs = {}
    for tag, L in libs.items():
        o = np.zeros(len(x_0) // 32 * 34, np.uint8)
        L.quantize_row_q8_0(ptr(x_0), ptr(o), len(x_0))
        outs[tag] = o
    assert np.array_equal(outs["avx2"], outs["avx512"]), "q8_0 quantizer differs between builds"
    G["q80_out"] = outs["avx2"]

    # ---- dequantizers on random valid blocks ------------------------------
    for fmt, fn in (("q4_k", "dequant_q4_k_row"), ("q6_k", "dequant_q6_k_row"), ("q8_0", "dequant_q8_0_row")):
        nblk = 6
        w = random_blocks(S, fmt, nblk, 200 + FMT[fmt])
        o = np.zeros(nblk * ELEMS[fmt], np.float32)
        getattr(libs["avx2"], fn)(ptr(w), ptr(o), ctypes.c_size_t(nblk * ELEMS[fmt]))
        G["deq_%s_w" % fmt] = w
        G["deq_%s_out" % fmt] = o

    # ---- GEMV / GEMM -------------------------------------------------------
    ROWS, K, TOK = 24, 1024, 3
    xf = normal(S, TOK * K, 0.0, 1.0, 301)
    G["act_f32"] = xf
    xq8k = np.zeros(TOK * (K // 256) * 292, np.uint8)
    libs["avx2"].quantize_batch_q8_k(ptr(xf), ptr(xq8k), TOK, K)
    G["act_q8k"] = xq8k
    xq80 = np.zeros(TOK * (K // 32) * 34, np.uint8)
    libs["avx2"].quantize_batch_q8_0(ptr(xf), ptr(xq80), TOK, K)
    G["act_q80"] = xq80
    # activation blocks whose stored bsums are zero: kernels must consume the
    # stored sums, not recompute them
    xz = xq8k.copy().reshape(-1, 292)
    xz[:, 260:292] = 0
    xz = xz.reshape(-1)
    G["act_q8k_zero_bsums"] = xz
    bias = normal(S, ROWS, 0.0, 0.5, 302)
    G["bias"] = bias
    G["shape"] = np.array([ROWS, K, TOK], np.int32)

    def run(L, name, *args):
        getattr(L, name)(*args)

    for kind in ("rand", "enc"):
        for fmt in ("q4_k", "q5_k", "q6_k", "q8_0"):
            if kind == "rand":
                w = random_blocks(S, fmt, ROWS * (K // ELEMS[fmt]), 400 + FMT[fmt])
            else:
                w = synth_weights(S, fmt, ROWS, K, 500 + FMT[fmt])
            G["w_%s_%s" % (fmt, kind)] = w
            act = xq80 if fmt == "q8_0" else xq8k
            gemv = {"q4_k": "gemv_q4_k_q8_k", "q5_k": "gemv_q5_k_q8_k",
                    "q6_k": "gemv_q6_k_q8_k", "q8_0": "gemv_q8_0_q8_0"}[fmt]
            gemm = {"q4_k": "gemm_nt_q4_k_q8_k", "q5_k": "gemm_nt_q5_k_q8_k",
                    "q6_k": "gemm_nt_q6_k_q8_k", "q8_0": "gemm_nt_q8_0_q8_0"}[fmt]
            for tag, L in libs.items():
                y = np.zeros(ROWS, np.float32)
                run(L, gemv, ptr(y), ptr(w), ptr(act), ROWS, K)
                G["y_%s_%s_%s" % (fmt, kind, tag)] = y
                c = np.zeros(TOK * ROWS, np.float32)
                run(L, gemm, ptr(act), ptr(w), ptr(bias), ptr(c), TOK, ROWS, K)
                G["c_%s_%s_%s" % (fmt, kind, tag)] = c
            if fmt == "q4_k":
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], "gemv_q4_k_q8_k_ref", ptr(y), ptr(w), ptr(act), ROWS, K)
                G["y_q4_k_%s_ref" % kind] = y
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], gemv, ptr(y), ptr(w), ptr(xz), ROWS, K)
                G["y_q4_k_%s_zero_bsums" % kind] = y
                y = np.zeros(ROWS, np.float32)
                for ith in range(5):
                    run(libs["avx2"], "gemv_q4_k_q8_k_parallel_simd", ptr(y), ptr(w), ptr(act), ROWS, K, ith, 5)
                G["y_q4_k_%s_parallel5" % kind] = y
            # fp32 activations, no activation quantization (both builds: they sum in different orders)
            if fmt in ("q4_k", "q6_k", "q8_0"):
                for tag, L in libs.items():
                    if fmt != "q8_0":
                        y = np.zeros(ROWS, np.float32)
                        run(L, "gemv_" + fmt, ptr(y), ptr(w), ptr(xf), ROWS, K)
                        G["y_%s_%s_f32w_%s" % (fmt, kind, tag)] = y
                    c = np.zeros(TOK * ROWS, np.float32)
                    run(L, "gemm_nt_" + fmt, ptr(xf), ptr(w), ptr(bias), ptr(c), TOK, ROWS, K)
                    G["c_%s_%s_f32w_%s" % (fmt, kind, tag)] = c
            if fmt == "q5_k":
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], gemv, ptr(y), ptr(w), ptr(xz), ROWS, K)
                G["y_q5_k_%s_zero_bsums" % kind] = y
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], "gemv_q5_k", ptr(y), ptr(w), ptr(xf), ROWS, K)
                G["y_q5_k_%s_f32act" % kind] = y
                c = np.zeros(TOK * ROWS, np.float32)
                run(libs["avx2"], "gemm_nt_q5_k", ptr(xf), ptr(w), ptr(bias), ptr(c), TOK, ROWS, K)
                G["c_q5_k_%s_f32act" % kind] = c
            if fmt == "q6_k":
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], "gemv_q6_k_q8_k_ref", ptr(y), ptr(w), ptr(act), ROWS, K)
                G["y_q6_k_%s_ref" % kind] = y
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], gemv, ptr(y), ptr(w), ptr(xz), ROWS, K)
                G["y_q6_k_%s_zero_bsums" % kind] = y
                s = np.zeros(1, np.float32)
                run(libs["avx2"], "vec_dot_q6_k_q8_k", K, ptr(s), ptr(w), ptr(act))
                G["s_q6_k_%s_vecdot" % kind] = s
            if fmt == "q8_0":
                y = np.zeros(ROWS, np.float32)
                run(libs["avx2"], "gemv_q8_0", ptr(y), ptr(w), ptr(xf), ROWS, K)
                G["y_q8_0_%s_f32act" % kind] = y
                s = np.zeros(1, np.float32)
                run(libs["avx2"], "vec_dot_q8_0_q8_0", K, ptr(s), ptr(w), ptr(act))
                G["s_q8_0_%s_vecdot" % kind] = s

    # ---- Q5_0 weights x Q8_0 activations (the fallback format of rows K-quants cannot hold) ----
    for kind in ("rand", "enc"):
        w = random_blocks(S, "q5_0", ROWS * (K // 32), 450) if kind == "rand" else synth_weights(S, "q5_0", ROWS, K, 550)
        G["w_q5_0_" + kind] = w
        for tag, L in libs.items():
            y = np.zeros(ROWS, np.float32)
            run(L, "gemv_q5_0_q8_0", ptr(y), ptr(w), ptr(xq80), ROWS, K)
            G["y_q5_0_%s_%s" % (kind, tag)] = y
            c = np.zeros(TOK * ROWS, np.float32)
            run(L, "gemm_nt_q5_0_q8_0", ptr(xq80), ptr(w), ptr(bias), ptr(c), TOK, ROWS, K)
            G["c_q5_0_%s_%s" % (kind, tag)] = c
        sv = np.zeros(1, np.float32)
        run(libs["avx2"], "vec_dot_q5_0_q8_0", K, ptr(sv), ptr(w), ptr(xq80))
        G["s_q5_0_%s_vecdot" % kind] = sv
        sv = np.zeros(1, np.float32)
        run(libs["avx2"], "vec_dot_q5_0_q8_0_ref", K, ptr(sv), ptr(w), ptr(xq80))
        G["s_q5_0_%s_vecdot_ref" % kind] = sv

    # ---- fused producer rmsnorm -> Q8_K (both builds must agree: integer output) ----
    TF, DF, AF = 3, 768, 800                       # row stride larger than d_model
    xr = normal(S, TF * AF, 0.0, 1.5, 601)
    xr.reshape(TF, AF)[1, 256:512] = 0.0           # a block of zeros -> zero block
    xr.reshape(TF, AF)[2, :] *= 40.0               # large magnitudes
    gam = normal(S, DF, 1.0, 0.4, 602)
    gam[5] = -gam[5]
    G["rms_in"], G["rms_gamma"] = xr, gam
    G["rms_shape"] = np.array([TF, DF, AF], np.int32)
    G["rms_eps"] = np.array([1e-6], np.float32)
    outs = {}
    for tag, L in libs.items():
        o = np.zeros(TF * (DF // 256) * 292, np.uint8)
        L.rmsnorm_q8_k_fused(ptr(xr), ptr(gam), ptr(o), TF, DF, AF, ctypes.c_float(1e-6))
        outs[tag] = o
    assert np.array_equal(outs["avx2"], outs["avx512"]), "rmsnorm_q8_k_fused differs between builds"
    G["rms_out"] = outs["avx2"]

    # ---- quantized embedding lookup ----------------------------------------------
    VOC, ED, AED, CTX, NTOK = 12, 500, 512, 7, 5
    ids = np.array([3, 11, -2, 40, 0], np.int32)            # two ids outside [0, VOC) -> row 0
    posv = normal(S, CTX * AED, 0.0, 0.1, 701)
    G["emb_ids"], G["emb_pos"] = ids, posv
    G["emb_shape"] = np.array([VOC, ED, AED, CTX, NTOK], np.int32)
    for fmt in ("q4_k", "q6_k", "q8_0"):
        tab = random_blocks(S, fmt, VOC * (AED // ELEMS[fmt]), 710 + FMT[fmt])
        G["emb_table_" + fmt] = tab
        for add_pos in (0, 1):
            o = np.full(CTX * AED, 9.0, np.float32)
            getattr(libs["avx2"], "embedding_forward_" + fmt)(ptr(ids), NTOK, VOC, ptr(tab), ptr(posv), ptr(o),
                                                               ED, AED, CTX, add_pos)
            G["emb_out_%s_pos%d" % (fmt, add_pos)] = o

    # ---- fused prefill MLP (Q8_0 gate/up, Q4_K or Q6_K down) -------------------------
    # 70 tokens: the reference walks tiles of 64, so the second tile is ragged
    SEQ, ED2, AED2, ID2, AID2 = 70, 60, 64, 250, 256
    xm = normal(S, SEQ * AED2, 0.0, 1.0, 801)
    w1 = synth_weights(S, "q8_0", 2 * AID2, AED2, 802)
    # synth weights are N(0, 0.02): scale the block scales up so gate values spread over the SiLU's knee
    w1v = w1.reshape(-1, 34)
    d16 = w1v[:, 0:2].copy().view(np.float16).astype(np.float32) * 12.0
    w1v[:, 0:2] = d16.astype(np.float16).view(np.uint8)
    b1 = normal(S, 2 * AID2, 0.0, 0.3, 803)
    b2 = normal(S, AED2, 0.0, 0.3, 804)
    G["mlp_x"], G["mlp_w1"], G["mlp_b1"], G["mlp_b2"] = xm, w1, b1, b2
    G["mlp_shape"] = np.array([SEQ, ED2, AED2, ID2, AID2], np.int32)
    DT = {"q4_k": 7, "q6_k": 8, "q8_0": 9}
    for fmt in ("q4_k", "q6_k"):
        w2 = synth_weights(S, fmt, AED2, AID2, 805 + FMT[fmt])
        G["mlp_w2_" + fmt] = w2
        for tag, L in libs.items():
            L.fused_mlp_swiglu_prefill_w1w2_quant_scratch_size.restype = ctypes.c_size_t
            scr = np.zeros(L.fused_mlp_swiglu_prefill_w1w2_quant_scratch_size(AED2, AID2), np.uint8)
            o = np.zeros(SEQ * AED2, np.float32)
            L.fused_mlp_swiglu_prefill_w1w2_quant(ptr(xm), ptr(w1), ptr(b1), DT["q8_0"], ptr(w2), ptr(b2), DT[fmt],
                                                  ptr(o), SEQ, ED2, AED2, ID2, AID2, ptr(scr))
            G["mlp_out_%s_%s" % (fmt, tag)] = o
        G["mlp_scratch_size"] = np.array([len(scr)], np.int64)
    # the same with the gate/up matrix in Q5_0
    w1q5 = synth_weights(S, "q5_0", 2 * AID2, AED2, 812)
    w1v = w1q5.reshape(-1, 22)
    d16 = w1v[:, 0:2].copy().view(np.float16).astype(np.float32) * 12.0
    w1v[:, 0:2] = d16.astype(np.float16).view(np.uint8)
    G["mlp_w1_q5_0"] = w1q5
    for tag, L in libs.items():
        scr = np.zeros(L.fused_mlp_swiglu_prefill_w1w2_quant_scratch_size(AED2, AID2), np.uint8)
        o = np.zeros(SEQ * AED2, np.float32)
        L.fused_mlp_swiglu_prefill_w1w2_quant(ptr(xm), ptr(w1q5), ptr(b1), 11, ptr(G["mlp_w2_q4_k"]), ptr(b2), DT["q4_k"],
                                              ptr(o), SEQ, ED2, AED2, ID2, AID2, ptr(scr))
        G["mlp_out_q5_0w1_q4_k_%s" % tag] = o

    np.savez_compressed(OUT, **G)
    print("wrote %s: %d arrays, %.1f KiB" % (OUT, len(G), os.path.getsize(OUT) / 1024.0))


if __name__ == "__main__":
    main()
