"""ctypes binding of libckernel_quant_hip.so (the C ABI declared in
include/ckernel_quant_hip.h) and of the host-side synthetic-data helper."""
import ctypes
import os
import re
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HEADER = os.path.join(ROOT, "include", "ckernel_quant_hip.h")

FMT = {"q4_k": 0, "q5_k": 1, "q6_k": 2, "q8_0": 3, "q8_k": 4, "q5_0": 5}
BLOCK_BYTES = {"q4_k": 144, "q5_k": 176, "q6_k": 210, "q8_0": 34, "q8_k": 292, "q5_0": 22}
BLOCK_ELEMS = {"q4_k": 256, "q5_k": 256, "q6_k": 256, "q8_0": 32, "q8_k": 256, "q5_0": 32}


class CkqError(RuntimeError):
    pass


def row_bytes(fmt, k):
    return (k // BLOCK_ELEMS[fmt]) * BLOCK_BYTES[fmt]


def lib_path():
    """The product library; CKQ_LIBRARY names another build of it to load instead (the UBSan
    build of the host layer, `make -C csrc ubsan`)."""
    return os.environ.get("CKQ_LIBRARY") or os.path.join(CSRC, "libckernel_quant_hip.so")


def dump_lib_path():
    """The test build of the same sources: every kernel also exists in a form that stores the
    integers behind its outputs (the exactness tests' entry points run only there)."""
    return os.path.join(CSRC, "libckernel_quant_hip_dump.so")


def build(targets=("synth", "hip", "dump")):
    """Compile the host helper and the gfx950 library in-tree (hipcc
    cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", CSRC, "-B"] + list(targets), check=True)


_c = ctypes
_vp, _i, _l, _f32p = _c.c_void_p, _c.c_int, _c.c_long, _c.c_void_p

# name -> (restype, argtypes); pointers are passed as integers / c_void_p so
# that host arrays and device addresses go through the same binding.
_SIGS = {
    "quantize_row_q8_k": (None, [_vp, _vp, _i]),
    "quantize_batch_q8_k": (None, [_vp, _vp, _i, _i]),
    "quantize_row_q8_0": (None, [_vp, _vp, _i]),
    "quantize_batch_q8_0": (None, [_vp, _vp, _i, _i]),
    "gemv_q4_k_q8_k": (None, [_vp, _vp, _vp, _i, _i]),
    "gemv_q4_k_q8_k_ref": (None, [_vp, _vp, _vp, _i, _i]),
    "gemv_q4_k_q8_k_parallel": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemv_q4_k_q8_k_parallel_simd": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemm_q4_k_q8_k": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "gemm_nt_q4_k_q8_k": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "gemv_q5_k_q8_k": (None, [_vp, _vp, _vp, _i, _i]),
    "gemm_nt_q5_k_q8_k": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "gemv_q5_k": (None, [_vp, _vp, _vp, _i, _i]),
    "gemm_nt_q5_k": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vec_dot_q6_k_q8_k": (None, [_i, _vp, _vp, _vp]),
    "gemv_q6_k_q8_k": (None, [_vp, _vp, _vp, _i, _i]),
    "gemv_q6_k_q8_k_parallel": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemv_q6_k_q8_k_parallel_simd": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemm_q6_k_q8_k": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "gemm_nt_q6_k_q8_k": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vec_dot_q8_0_q8_0": (None, [_i, _vp, _vp, _vp]),
    "gemv_q8_0_q8_0": (None, [_vp, _vp, _vp, _i, _i]),
    "gemv_q8_0_q8_0_parallel": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemv_q8_0_q8_0_parallel_simd": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemv_q8_0": (None, [_vp, _vp, _vp, _i, _i]),
    "gemm_nt_q8_0_q8_0": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "dequant_q4_k_row": (None, [_vp, _vp, _c.c_size_t]),
    "dequant_q6_k_row": (None, [_vp, _vp, _c.c_size_t]),
    "dequant_q8_0_row": (None, [_vp, _vp, _c.c_size_t]),
    "embedding_forward_q4_k": (None, [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i]),
    "embedding_forward_q6_k": (None, [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i]),
    "embedding_forward_q8_0": (None, [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i]),
    "rmsnorm_q8_k_fused": (None, [_vp, _vp, _vp, _i, _i, _i, _c.c_float]),
    "vec_dot_q5_0_q8_0": (None, [_i, _vp, _vp, _vp]),
    "gemv_q5_0_q8_0": (None, [_vp, _vp, _vp, _i, _i]),
    "gemv_q5_0_q8_0_parallel_simd": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "gemm_nt_q5_0_q8_0": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "fused_mlp_swiglu_prefill_w1w2_quant": (None, [_vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp]),
    "fused_mlp_swiglu_prefill_w1w2_quant_scratch_size": (_c.c_size_t, [_i, _i]),
    "gemv_q4_k": (None, [_vp, _vp, _vp, _i, _i]),
    "gemm_q4_k": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "gemm_nt_q4_k": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "dot_q4_k": (_c.c_float, [_vp, _vp, _i]),
    "gemv_q6_k": (None, [_vp, _vp, _vp, _i, _i]),
    "gemm_q6_k": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "gemm_nt_q6_k": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "gemm_q8_0": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "gemm_nt_q8_0": (None, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "ck_test_quantize_q8_k": (None, [_vp, _vp, _i]),
    "ck_test_dequant_q4_k": (None, [_vp, _vp, _i]),
    "ck_test_dequant_q6_k": (None, [_vp, _vp, _i]),
    "ck_test_gemv_q4_k": (None, [_vp, _vp, _vp, _i]),
    "ck_test_gemv_q6_k": (None, [_vp, _vp, _vp, _i]),
    "ck_test_gemv_q8_0": (None, [_vp, _vp, _vp, _i, _i]),
    "ck_test_gemv_q8_0_q8_0": (None, [_vp, _vp, _vp, _i, _i]),
    "ck_test_vec_dot_q8_0_q8_0": (None, [_vp, _vp, _vp, _i]),
    "ck_test_gemm_q4_k": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "ck_test_gemm_q6_k": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "ck_test_gemm_q8_0": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "ck_get_block_q4_k_size": (_i, []),
    "ck_get_block_q6_k_size": (_i, []),
    "ck_get_block_q8_k_size": (_i, []),
    "ck_get_qk_k": (_i, []),
    "ckq_quantize_q8_k_dev": (_i, [_vp, _vp, _i, _i, _vp]),
    "ckq_quantize_q8_0_dev": (_i, [_vp, _vp, _i, _i, _vp]),
    "ckq_gemm_nt_dev": (_i, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _l, _vp]),
    "ckq_gemm_nt_noalloc_dev": (_i, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _l, _vp]),
    "ckq_gemv_q4_k_q8_k_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "ckq_gemv_q5_k_q8_k_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "ckq_gemv_q6_k_q8_k_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "ckq_gemv_q8_0_q8_0_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "ckq_gemv_q8_0_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "ckq_gemm_nt_q4_k_q8_k_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "ckq_gemm_nt_q5_k_q8_k_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "ckq_gemm_nt_q6_k_q8_k_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "ckq_gemm_nt_q8_0_q8_0_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "ckq_dequant_rows_dev": (_i, [_i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp]),
    "ckq_rmsnorm_q8_k_fused_dev": (_i, [_vp, _vp, _vp, _i, _i, _i, _c.c_float, _vp]),
    "ckq_swiglu_q8_k_dev": (_i, [_vp, _vp, _vp, _i, _i, _c.c_long, _vp]),
    "ckq_gemm_nt_f32act_dev": (_i, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _c.c_long, _vp]),
    "ckq_matmul_sequence_dev": (_i, [_vp, _i, _i, _vp]),
    "ckq_subblock_dots_dev": (_i, [_i, _vp, _vp, _vp, _i, _i, _vp]),
    "ckq_subblock_dots_tokens_dev": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "ckq_subblock_dots_group_dev": (_i, [_i, _i, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "ckq_gemm_block_sums_dev": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "ckq_copy_dev": (_i, [_vp, _vp, _c.c_size_t, _vp]),
    "ckq_read_dev": (_i, [_vp, _c.c_size_t, _vp, _vp]),
    "ckq_read_tuned_dev": (_i, [_vp, _c.c_size_t, _vp, _i, _i, _vp]),
    "ckq_init": (_i, []),
    "ckq_synchronize": (_i, []),
    "ckq_weights_register": (_i, [_vp, _c.c_size_t]),
    "ckq_weights_register_manifest": (_i, [_vp, _c.c_char_p]),
    "ckq_weights_resident": (_i, [_vp]),
    "ckq_weights_invalidate": (None, [_vp]),
    "ckq_weights_clear": (None, []),
    "ckq_weights_set_cache": (None, [_i]),
    "ckq_weights_set_limit": (None, [_c.c_size_t]),
    "ckq_release_stream": (_i, [_vp]),
    "ckq_set_parallel_whole": (None, [_i]),
    "ckq_set_prefill_grouping": (None, [_i]),
    "ckq_set_gemm_policy": (None, [_i]),
    "ckq_set_prefill_variant": (None, [_i, _i]),
    "ckq_last_error": (_i, []),
    "ckq_clear_error": (None, []),
    "ckq_error_string": (_c.c_char_p, [_i]),
}



class MatmulOp(ctypes.Structure):
    """ckq_matmul_op of include/ckernel_quant_hip.h."""
    _fields_ = [("fmt", _i), ("M", _i), ("N", _i), ("K", _i), ("ldc", _l),
                ("A_q8", _vp), ("B", _vp), ("bias", _vp), ("C", _vp), ("eps", _c.c_float)]


STEP = {"quantize_q8_k": 32, "quantize_q8_0": 33, "rmsnorm_q8_k": 34, "swiglu_q8_k": 35}


_lib = None
_synth = None


def declared_symbols():
    """Function names declared in include/ckernel_quant_hip.h."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"typedef\s+struct\s*\{.*?\}\s*\w+;", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?(?:void|int|char|float|size_t)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def lib():
    """The gfx950 library.  Raises CkqError if it has not been built: there is
    no fallback implementation."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise CkqError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                           "(there is no CPU fallback)" % path)
        L = ctypes.CDLL(path)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


_dump = None


def dump_lib():
    """The library with the integer-dump instantiations (test infrastructure; the product
    library answers the dump entry points with CKQ_ENODUMP)."""
    global _dump
    if _dump is None:
        path = dump_lib_path()
        if not os.path.exists(path):
            raise CkqError("%s is missing: build it with `make -C %s dump`" % (path, CSRC))
        L = ctypes.CDLL(path)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _dump = L
    return _dump


def synth_lib():
    """Host-side synthetic-data generator and weight encoders."""
    global _synth
    if _synth is None:
        path = os.path.join(CSRC, "libckq_synth.so")
        if not os.path.exists(path):
            raise CkqError("%s is missing: build it with `make -C %s synth`" % (path, CSRC))
        _synth = ctypes.CDLL(path)
    return _synth


def check(rc, what):
    if rc != 0:
        raise CkqError("%s failed: %s (%d)" % (what, lib().ckq_error_string(rc).decode(), rc))
