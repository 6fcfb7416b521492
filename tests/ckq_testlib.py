"""Shared helpers for the test-suite: ctypes handles to the CPU oracle and the
synthetic-data generator, NumPy block decoders written from the format
definitions (independent of the oracle's C code), and error metrics."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
ORACLE_DIR = os.path.join(ROOT, "oracle")
CSRC = os.path.join(ROOT, "c-kernel-engine_amd", "csrc")
GOLDEN = os.path.join(ROOT, "tests", "golden", "quant_path_golden.npz")

FMT = {"q4_k": 0, "q5_k": 1, "q6_k": 2, "q8_0": 3, "q8_k": 4, "q5_0": 5}
BLK = {"q4_k": 144, "q5_k": 176, "q6_k": 210, "q8_0": 34, "q8_k": 292, "q5_0": 22}
ELEMS = {"q4_k": 256, "q5_k": 256, "q6_k": 256, "q8_0": 32, "q8_k": 256, "q5_0": 32}

vp = ctypes.c_void_p


def ptr(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(vp)


def row_bytes(fmt, k):
    return (k // ELEMS[fmt]) * BLK[fmt]


def act_fmt(wfmt):
    return "q8_0" if wfmt in ("q8_0", "q5_0") else "q8_k"


_cache = {}


def _make(target_dir, target=None):
    cmd = ["make", "-s", "-C", target_dir]
    if target:
        cmd.append(target)
    subprocess.run(cmd, check=True)


def oracle():
    """CPU oracle (deterministic build)."""
    if "oracle" not in _cache:
        path = os.path.join(ORACLE_DIR, "libckq_oracle.so")
        if not os.path.exists(path):
            _make(ORACLE_DIR, "oracle")
        L = ctypes.CDLL(path)
        L.orc_fp16_to_fp32.restype = ctypes.c_float
        L.orc_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        L.orc_fp32_to_fp16.restype = ctypes.c_uint16
        L.orc_fp32_to_fp16.argtypes = [ctypes.c_float]
        _cache["oracle"] = L
    return _cache["oracle"]


def synth():
    if "synth" not in _cache:
        path = os.path.join(CSRC, "libckq_synth.so")
        if not os.path.exists(path):
            _make(CSRC, "synth")
        _cache["synth"] = ctypes.CDLL(path)
    return _cache["synth"]


def golden():
    if "golden" not in _cache:
        _cache["golden"] = np.load(GOLDEN, allow_pickle=False)
    return _cache["golden"]


# ---- synthetic inputs -------------------------------------------------------

def normal(n, mean=0.0, std=1.0, seed=1):
    out = np.empty(n, dtype=np.float32)
    synth().ckq_synth_normal(ptr(out), ctypes.c_size_t(n), ctypes.c_float(mean), ctypes.c_float(std),
                             ctypes.c_uint64(seed))
    return out


def synth_weights(fmt, rows, k, seed, std=0.02):
    out = np.zeros(rows * row_bytes(fmt, k), dtype=np.uint8)
    rc = synth().ckq_synth_weights(FMT[fmt], ptr(out), rows, k, ctypes.c_float(0.0), ctypes.c_float(std),
                                   ctypes.c_uint64(seed))
    assert rc == 0
    return out


def random_blocks(fmt, nblocks, seed):
    out = np.zeros(nblocks * BLK[fmt], dtype=np.uint8)
    rc = synth().ckq_synth_random_blocks(FMT[fmt], ptr(out), ctypes.c_size_t(nblocks), ctypes.c_uint64(seed))
    assert rc == 0
    return out


def oracle_quantize(x, fmt="q8_k", rows=1):
    """fp32 [rows*k] -> activation blocks, through the oracle."""
    k = len(x) // rows
    out = np.zeros(rows * row_bytes(fmt, k), dtype=np.uint8)
    fn = oracle().orc_quantize_batch_q8_k if fmt == "q8_k" else oracle().orc_quantize_batch_q8_0
    fn(ptr(x), ptr(out), rows, k)
    return out


ORC_GEMV = {"q4_k": "orc_gemv_q4_k_q8_k", "q5_k": "orc_gemv_q5_k_q8_k",
            "q6_k": "orc_gemv_q6_k_q8_k", "q8_0": "orc_gemv_q8_0_q8_0", "q5_0": "orc_gemv_q5_0_q8_0"}
ORC_GEMM_NT = {"q4_k": "orc_gemm_nt_q4_k_q8_k", "q5_k": "orc_gemm_nt_q5_k_q8_k",
               "q6_k": "orc_gemm_nt_q6_k_q8_k", "q8_0": "orc_gemm_nt_q8_0_q8_0", "q5_0": "orc_gemm_nt_q5_0_q8_0"}
ORC_SUBDOTS = {"q4_k": ("orc_subdots_q4_k_q8_k", 8), "q5_k": ("orc_subdots_q5_k_q8_k", 8),
               "q6_k": ("orc_subdots_q6_k_q8_k", 16), "q8_0": ("orc_subdots_q8_0_q8_0", 1),
               "q5_0": ("orc_subdots_q5_0_q8_0", 1)}


def oracle_gemv(fmt, W, xq, M, K, name=None):
    y = np.zeros(M, dtype=np.float32)
    getattr(oracle(), name or ORC_GEMV[fmt])(ptr(y), ptr(W), ptr(xq), M, K)
    return y


def oracle_gemm_nt(fmt, A, B, bias, M, N, K):
    c = np.zeros(M * N, dtype=np.float32)
    getattr(oracle(), ORC_GEMM_NT[fmt])(ptr(A), ptr(B), ptr(bias) if bias is not None else None, ptr(c), M, N, K)
    return c.reshape(M, N)


def oracle_gemm_nt_f32act(fmt, A_f32, B, bias, M, N, K):
    """fp32 activations, nothing quantized (orc_gemm_nt_q4_k / _q6_k / _q8_0)."""
    c = np.zeros(M * N, dtype=np.float32)
    getattr(oracle(), "orc_gemm_nt_" + fmt)(ptr(A_f32), ptr(B), ptr(bias) if bias is not None else None, ptr(c), M, N, K)
    return c.reshape(M, N)


CK_DT = {"q4_k": 7, "q6_k": 8, "q8_0": 9, "q8_k": 10, "q5_0": 11}   # the reference's CKDataType values


def oracle_fused_mlp(x, W1, B1, W2, B2, w2_fmt, seq, embed, aembed, inter, ainter, want_intermediates=False, w1_fmt="q8_0"):
    out = np.zeros(seq * aembed, dtype=np.float32)
    gu = np.zeros(seq * 2 * ainter, dtype=np.float32) if want_intermediates else None
    hq = np.zeros(seq * row_bytes("q8_k", ainter), dtype=np.uint8) if want_intermediates else None
    oracle().orc_fused_mlp_swiglu_prefill_w1w2_quant(ptr(x), ptr(W1), ptr(B1), CK_DT[w1_fmt], ptr(W2), ptr(B2),
                                                     CK_DT[w2_fmt], ptr(out), seq, embed, aembed, inter, ainter,
                                                     ptr(gu), ptr(hq))
    out = out.reshape(seq, aembed)
    return (out, gu.reshape(seq, 2 * ainter), hq) if want_intermediates else out


def oracle_exact(fmt, W, xq, M, K):
    y = np.zeros(M, dtype=np.float64)
    oracle().orc_gemv_exact_f64(FMT[fmt], ptr(y), ptr(W), ptr(xq), M, K)
    return y


def oracle_subdots(fmt, W, xq, M, K):
    name, per = ORC_SUBDOTS[fmt]
    nsub = (K // ELEMS[fmt]) * per
    out = np.zeros((M, nsub), dtype=np.int32)
    rb = row_bytes(fmt, K)
    for r in range(M):
        getattr(oracle(), name)(ptr(W[r * rb:(r + 1) * rb]), ptr(xq), K, ptr(out[r]))
    return out


# ---- NumPy block decoders (from the format definitions) ----------------------

def _f16(b):
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)


def np_scales_k4(s12):
    """[n,12] packed bytes -> ([n,8] scales, [n,8] mins)."""
    s = s12.astype(np.uint8)
    sc = np.zeros(s.shape[:-1] + (8,), np.uint8)
    mn = np.zeros_like(sc)
    sc[..., :4] = s[..., 0:4] & 63
    mn[..., :4] = s[..., 4:8] & 63
    sc[..., 4:] = (s[..., 8:12] & 15) | ((s[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, mn


def np_decode_q4_k(w):
    """bytes -> dict(d, dmin [n], sc, mn [n,8], q [n,256] in element order)."""
    b = w.reshape(-1, 144)
    d = _f16(b[:, 0:2]).reshape(-1)
    dmin = _f16(b[:, 2:4]).reshape(-1)
    sc, mn = np_scales_k4(b[:, 4:16])
    qs = b[:, 16:144].reshape(-1, 4, 32)
    q = np.concatenate([qs & 15, qs >> 4], axis=2).reshape(-1, 256)  # per 64-group: 32 low then 32 high
    return dict(d=d, dmin=dmin, sc=sc, mn=mn, q=q.astype(np.int32))


def np_decode_q5_k(w):
    b = w.reshape(-1, 176)
    d = _f16(b[:, 0:2]).reshape(-1)
    dmin = _f16(b[:, 2:4]).reshape(-1)
    sc, mn = np_scales_k4(b[:, 4:16])
    qh = b[:, 16:48]                       # [n,32]
    qs = b[:, 48:176].reshape(-1, 4, 32)
    out = np.zeros((b.shape[0], 4, 64), np.int32)
    for g in range(4):
        out[:, g, :32] = (qs[:, g] & 15) | (((qh >> (2 * g)) & 1) << 4)
        out[:, g, 32:] = (qs[:, g] >> 4) | (((qh >> (2 * g + 1)) & 1) << 4)
    return dict(d=d, dmin=dmin, sc=sc, mn=mn, q=out.reshape(-1, 256))


def np_decode_q6_k(w):
    b = w.reshape(-1, 210)
    ql = b[:, 0:128].reshape(-1, 2, 64)
    qh = b[:, 128:192].reshape(-1, 2, 32)
    sc = b[:, 192:208].view(np.int8).astype(np.int32)
    d = _f16(b[:, 208:210]).reshape(-1)
    out = np.zeros((b.shape[0], 2, 128), np.int32)
    for n in range(2):
        lo0, lo1, h = ql[:, n, :32].astype(np.int32), ql[:, n, 32:].astype(np.int32), qh[:, n].astype(np.int32)
        out[:, n, 0:32] = ((lo0 & 15) | ((h & 3) << 4)) - 32
        out[:, n, 32:64] = ((lo1 & 15) | (((h >> 2) & 3) << 4)) - 32
        out[:, n, 64:96] = ((lo0 >> 4) | (((h >> 4) & 3) << 4)) - 32
        out[:, n, 96:128] = ((lo1 >> 4) | (((h >> 6) & 3) << 4)) - 32
    return dict(d=d, sc=sc, q=out.reshape(-1, 256))


def np_decode_q8_0(w):
    b = w.reshape(-1, 34)
    return dict(d=_f16(b[:, 0:2]).reshape(-1), q=b[:, 2:34].view(np.int8).astype(np.int32))


def np_decode_q5_0(w):
    """From the format definition: element l < 16 = low nibble of qs[l] | bit l of
    qh << 4, element 16 + l = high nibble | bit 16 + l << 4; value = q - 16."""
    b = w.reshape(-1, 22)
    qh = np.ascontiguousarray(b[:, 2:6]).view(np.uint32).reshape(-1).astype(np.int64)
    qs = b[:, 6:22].astype(np.int32)
    bits = ((qh[:, None] >> np.arange(32)[None, :]) & 1).astype(np.int32)
    q = np.concatenate([qs & 15, qs >> 4], axis=1) | (bits << 4)
    return dict(d=_f16(b[:, 0:2]).reshape(-1), q=q - 16)


def np_decode_q8_k(x):
    b = x.reshape(-1, 292)
    return dict(d=np.ascontiguousarray(b[:, 0:4]).view(np.float32).reshape(-1),
                q=b[:, 4:260].view(np.int8).astype(np.int32),
                bsums=np.ascontiguousarray(b[:, 260:292]).view(np.int16).astype(np.int32))


def np_dequant(fmt, w):
    """bytes -> float64 element values."""
    if fmt in ("q4_k", "q5_k"):
        b = np_decode_q4_k(w) if fmt == "q4_k" else np_decode_q5_k(w)
        q = b["q"].reshape(-1, 8, 32).astype(np.float64)
        step = (b["d"][:, None].astype(np.float64) * b["sc"])[:, :, None]
        off = (b["dmin"][:, None].astype(np.float64) * b["mn"])[:, :, None]
        return (step * q - off).reshape(-1)
    if fmt == "q6_k":
        b = np_decode_q6_k(w)
        q = b["q"].reshape(-1, 16, 16).astype(np.float64)
        return (b["d"][:, None, None].astype(np.float64) * b["sc"][:, :, None] * q).reshape(-1)
    if fmt in ("q8_0", "q5_0"):
        b = np_decode_q8_0(w) if fmt == "q8_0" else np_decode_q5_0(w)
        return (b["d"][:, None].astype(np.float64) * b["q"]).reshape(-1)
    if fmt == "q8_k":
        b = np_decode_q8_k(w)
        return (b["d"][:, None].astype(np.float64) * b["q"]).reshape(-1)
    raise ValueError(fmt)


def np_subdots(fmt, W, xq, M, K):
    """Brute-force integer sub-block dots, [M, nsub]."""
    if fmt in ("q8_0", "q5_0"):
        wq = (np_decode_q8_0(W) if fmt == "q8_0" else np_decode_q5_0(W))["q"].reshape(M, K // 32, 32)
        xv = np_decode_q8_0(xq)["q"].reshape(K // 32, 32)
        return (wq * xv[None]).sum(axis=2).astype(np.int32)
    xv = np_decode_q8_k(xq)["q"].reshape(K // 256, 256)
    dec = {"q4_k": np_decode_q4_k, "q5_k": np_decode_q5_k, "q6_k": np_decode_q6_k}[fmt](W)
    wq = dec["q"].reshape(M, K // 256, 256)
    sub = 16 if fmt == "q6_k" else 32
    prod = (wq * xv[None]).reshape(M, K // 256, 256 // sub, sub).sum(axis=3)
    return prod.reshape(M, -1).astype(np.int32)


def norm_err(y, ref):
    """max|y-ref| / max|ref| : the normalised error the parity bar uses."""
    y = np.asarray(y, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    den = np.max(np.abs(ref))
    return float(np.max(np.abs(y - ref)) / den) if den > 0 else float(np.max(np.abs(y - ref)))


# ---- the reference's thread pool as caller -------------------------------------------

POOL_LIB = os.path.join(ORACLE_DIR, "_ref", "libckref_pool.so")


def ref_pool(kernel_lib_path):
    """The reference's thread pool + parallel decode dispatch (oracle/_ref/libckref_pool.so,
    built from the reference's ck_threadpool.c, ckernel_strict.c and ck_parallel_decode.c),
    with its undefined kernel symbols bound to the library at `kernel_lib_path`.

    That library is (re)opened RTLD_GLOBAL first; the pool library is opened with lazy
    binding, because it also names kernels that no quantized-path library defines and
    that are never called here (ctypes itself always binds eagerly).  Returns None when
    the pool library has not been built (no reference checkout at build time)."""
    if not os.path.exists(POOL_LIB):
        return None
    key = "pool:" + kernel_lib_path
    if key not in _cache:
        ctypes.CDLL(kernel_lib_path, mode=ctypes.RTLD_GLOBAL)
        libc = ctypes.CDLL(None)
        libc.dlopen.restype = ctypes.c_void_p
        libc.dlopen.argtypes = [ctypes.c_char_p, ctypes.c_int]
        handle = libc.dlopen(POOL_LIB.encode(), os.RTLD_LAZY | os.RTLD_GLOBAL)
        if not handle:
            raise OSError("dlopen(%s) failed" % POOL_LIB)
        L = ctypes.CDLL(POOL_LIB, handle=handle)
        for name in ("gemv_q4_k_q8_k_parallel_dispatch", "gemv_q6_k_q8_k_parallel_dispatch",
                     "gemv_q8_0_q8_0_parallel_dispatch", "gemv_q5_k_parallel_dispatch"):
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = [vp, vp, vp, ctypes.c_int, ctypes.c_int]
        L.ck_set_num_threads.argtypes = [ctypes.c_int]
        L.ck_threadpool_global.restype = vp
        L.ck_threadpool_n_threads.argtypes = [vp]
        _cache[key] = L
    return _cache[key]


def ref_pool_set_threads(pool, n):
    """Recreate the reference's global pool with n threads."""
    pool.ck_threadpool_global_destroy()
    pool.ck_set_num_threads(n)
    assert pool.ck_threadpool_n_threads(pool.ck_threadpool_global()) == n
