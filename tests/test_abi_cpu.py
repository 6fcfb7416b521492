"""CPU checks of the C-ABI library: it loads, exports every declared symbol,
and the host logic that needs no device (argument screening) behaves like the
reference.  No kernel is launched here."""
import ctypes
import importlib
import os
import subprocess

import numpy as np
import pytest

ckq = importlib.import_module("c-kernel-engine_amd")


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(ckq.lib_path()):
        ckq.build()
    return ckq.lib()


def test_every_declared_symbol_is_exported(L):
    names = ckq.declared_symbols()
    assert len(names) >= 60
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    # and the binding table covers the header
    from importlib import import_module
    api = import_module("c-kernel-engine_amd.api")
    assert sorted(api._SIGS) == names


def test_reference_symbol_names_present(L):
    # the symbols a generated libmodel.so resolves for this path
    # (reference include/ckernel_engine.h:192-363)
    for n in ["quantize_row_q8_k", "quantize_batch_q8_k", "quantize_row_q8_0", "gemv_q4_k_q8_k",
              "gemv_q4_k_q8_k_parallel_simd", "gemm_nt_q4_k_q8_k", "gemv_q5_k", "gemm_nt_q5_k",
              "gemv_q6_k_q8_k", "gemv_q6_k_q8_k_parallel_simd", "gemm_nt_q6_k_q8_k", "gemv_q8_0_q8_0",
              "gemv_q8_0", "gemm_nt_q8_0_q8_0", "vec_dot_q6_k_q8_k", "vec_dot_q8_0_q8_0"]:
        assert hasattr(L, n)
    # the parity scripts' wrappers (reference include/ck_parity_api.h:42-56, 193-201)
    for n in ["ck_test_dequant_q4_k", "ck_test_dequant_q6_k", "ck_test_quantize_q8_k", "ck_test_gemv_q4_k",
              "ck_test_gemv_q6_k", "ck_test_gemm_q4_k", "ck_test_gemm_q6_k", "ck_test_gemm_q8_0"]:
        assert hasattr(L, n)


def test_block_size_getters(L):
    assert L.ck_get_block_q4_k_size() == 144
    assert L.ck_get_block_q6_k_size() == 210
    assert L.ck_get_block_q8_k_size() == 292
    assert L.ck_get_qk_k() == 256


def test_bad_arguments_return_without_touching_output(L):
    """NULL pointer or non-positive dimension: silent return
    (reference gemm_kernels_q4k_q8k.c:188-190, :221-223, :307-312)."""
    y = np.full(8, 7.0, np.float32)
    w = np.zeros(8 * 144, np.uint8)
    x = np.zeros(292, np.uint8)
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    L.gemv_q4_k_q8_k(p(y), None, p(x), 8, 256)
    L.gemv_q4_k_q8_k(p(y), p(w), None, 8, 256)
    L.gemv_q4_k_q8_k(p(y), p(w), p(x), 0, 256)
    L.gemv_q4_k_q8_k(p(y), p(w), p(x), 8, -256)
    L.gemv_q4_k_q8_k_parallel(p(y), p(w), p(x), 8, 256, 3, 3)   # ith >= nth
    L.gemv_q4_k_q8_k_parallel(p(y), p(w), p(x), 8, 256, -1, 3)
    L.gemv_q4_k_q8_k_parallel_simd(p(y), p(w), p(x), 8, 256, 0, 0)
    L.gemv_q6_k_q8_k_parallel(p(y), p(w), p(x), 8, 256, 5, 2)
    L.gemv_q8_0_q8_0_parallel_simd(p(y), p(w), p(x), 8, 256, 2, 2)
    L.gemm_nt_q4_k_q8_k(None, p(w), None, p(y), 1, 8, 256)
    L.gemm_nt_q6_k_q8_k(p(x), p(w), None, p(y), 1, 0, 256)
    L.gemv_q5_k_q8_k(p(y), p(w), p(x), 8, 200)                   # K % 256 != 0 (gemm_kernels_q5_k.c:313-315)
    L.vec_dot_q6_k_q8_k(0, p(y), p(w), p(x))
    L.quantize_row_q8_k(None, p(x), 256)
    L.quantize_row_q8_k(p(y), p(x), 0)
    assert np.all(y == 7.0)
    assert L.ckq_last_error() == 0


def test_dev_entry_points_reject_bad_shapes(L):
    # status codes come back before anything touches a device
    one = ctypes.c_void_p(16)
    assert L.ckq_gemv_q4_k_q8_k_dev(one, one, one, 4, 100, None) == -2
    assert L.ckq_gemv_q4_k_q8_k_dev(None, one, one, 4, 256, None) == -1
    assert L.ckq_gemm_nt_dev(9, one, one, None, one, 1, 4, 256, 4, None) == -3
    assert L.ckq_quantize_q8_k_dev(one, one, 1, 100, None) == -2
    assert L.ckq_quantize_q8_0_dev(one, one, 0, 32, None) == -1
    assert b"multiple" in L.ckq_error_string(-2)


def test_manifest_hook_parses_without_touching_a_device(L, tmp_path):
    """The loader hook reads the reference's manifest format; tensors of other
    dtypes are skipped, so a manifest without quantized weights needs no device;
    unreadable files and malformed lines are reported as argument errors."""
    base = np.zeros(64, np.uint8)
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    m = tmp_path / "weights_manifest.map"
    m.write_text("# name|dtype|file_offset|size|runtime_offset\n\n"
                 "model.norm.weight|fp32|8|3584|0\n"
                 "model.rope.cache|f16|0x1000|128|4096\n")
    assert L.ckq_weights_register_manifest(p(base), str(m).encode()) == 0
    assert L.ckq_weights_register_manifest(p(base), str(tmp_path / "missing.map").encode()) == -1
    assert L.ckq_weights_register_manifest(None, str(m).encode()) == -1
    bad = tmp_path / "bad.map"
    bad.write_text("model.norm.weight|fp32|8|3584\n")
    assert L.ckq_weights_register_manifest(p(base), str(bad).encode()) == -1
    assert L.ckq_last_error() == 0
    nbytes = ctypes.c_size_t(7)
    assert L.ckq_weights_resident(ctypes.byref(nbytes)) == 0 and nbytes.value == 0


def test_header_compiles_next_to_the_reference_headers(tmp_path):
    """One translation unit with the reference's own headers and this library's:
    every shared prototype must be declaration-compatible (the fused MLP takes
    the reference's CKDataType, include/ckernel_engine.h:666-680)."""
    ref_inc = "/root/reference/include"
    if not os.path.exists(os.path.join(ref_inc, "ckernel_engine.h")):
        pytest.skip("reference checkout not present")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "tu.c"
    src.write_text('#include "ckernel_engine.h"\n#include "ckernel_quant.h"\n#include "ck_parity_api.h"\n'
                   '#include "ckernel_quant_hip.h"\n'
                   'void (*p)(const float *, const void *, const float *, CKDataType, const void *, const float *,\n'
                   '          CKDataType, float *, int, int, int, int, int, void *) = fused_mlp_swiglu_prefill_w1w2_quant;\n'
                   'int main(void) { return 0; }\n')
    r = subprocess.run(["gcc", "-std=gnu11", "-Wall", "-Werror", "-I" + ref_inc, "-I" + os.path.join(root, "include"),
                        "-c", str(src), "-o", str(tmp_path / "tu.o")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    # and on its own, as C and as C++
    alone = tmp_path / "alone.c"
    alone.write_text('#include "ckernel_quant_hip.h"\nint main(void) { return (int)sizeof(ckq_ck_dtype) - 4; }\n')
    for cc, std in (("gcc", "-std=gnu11"), ("g++", "-std=c++17")):
        r = subprocess.run([cc, std, "-Wall", "-Werror", "-x", "c" if cc == "gcc" else "c++",
                            "-I" + os.path.join(root, "include"), "-c", str(alone), "-o", str(tmp_path / "a.o")],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr


def test_grid_chunk_index_arithmetic(L):
    """Launches whose token tiles exceed gridDim.y's 65 535 are issued in chunks;
    the chunks must tile [0, total) exactly, in order, without overlap."""
    L.ckq_grid_chunk.restype = None
    L.ckq_grid_chunk.argtypes = [ctypes.c_long] * 3 + [ctypes.POINTER(ctypes.c_long)] * 2
    for total, per in ((1, 65535), (65535, 65535), (65536, 65535), (70000, 65535), (131072, 65535),
                       (8 * 65535 + 3, 8 * 65535), (200000, 2 * 65535)):
        covered, c = 0, 0
        while c * per < total:
            first, count = ctypes.c_long(), ctypes.c_long()
            L.ckq_grid_chunk(total, per, c, ctypes.byref(first), ctypes.byref(count))
            assert first.value == covered and 0 < count.value <= per
            covered += count.value
            c += 1
        assert covered == total and c == -(-total // per)


def test_workspace_slot_bookkeeping(L):
    """Slot choice of the per-(device, stream, kind) scratch table of the K-split
    GEMMs: a known key finds its slot, a new key takes the first free slot, and
    with every slot taken the least recently used one is handed out for
    recycling - more distinct streams than slots must not fail."""
    n = 8
    U64 = ctypes.c_uint64 * n
    L.ckq_workspace_pick.restype = ctypes.c_int
    L.ckq_workspace_pick.argtypes = [U64, U64, ctypes.c_int, ctypes.c_uint64]
    keys, use = U64(), U64()
    clock = 0
    where = {}
    for k in range(1, 3 * n + 1):                    # 24 distinct "streams" through 8 slots
        key = (1 << 63) | (0x7f0000001000 + 64 * k)
        i = L.ckq_workspace_pick(keys, use, n, key)
        assert 0 <= i < n
        if k <= n:
            assert keys[i] == 0 and i == k - 1       # first free slot, in order
        else:
            assert use[i] == min(use)                # least recently used
            where = {kk: ii for kk, ii in where.items() if ii != i}
        keys[i] = key
        clock += 1
        use[i] = clock
        where[key] = i
        # a key that is present is found again, whatever its age
        for kk, ii in where.items():
            assert L.ckq_workspace_pick(keys, use, n, kk) == ii
    # touching an old entry protects it from being the next victim
    oldest = min(range(n), key=lambda j: use[j])
    clock += 1
    use[oldest] = clock
    assert L.ckq_workspace_pick(keys, use, n, (1 << 63) | 0x1234) != oldest


def test_no_device_fails_loudly():
    """Without a GPU a compute call must not succeed silently: the library
    reports the HIP error and aborts the process."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    code = (
        "import importlib, numpy as np, ctypes\n"
        "ckq = importlib.import_module('c-kernel-engine_amd')\n"
        "x = np.ones(256, np.float32); y = np.zeros(292, np.uint8)\n"
        "ckq.lib().quantize_row_q8_k(x.ctypes.data_as(ctypes.c_void_p), y.ctypes.data_as(ctypes.c_void_p), 256)\n"
        "print('survived')\n"
    )
    r = subprocess.run(["python", "-c", code], capture_output=True, text=True,
                       cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode != 0
    assert "survived" not in r.stdout
    assert "no CPU fallback" in r.stderr


def test_dpp_hazard_checker(tmp_path):
    """csrc/check_dpp.py, the build's check of the GEMMs' hand-written DPP
    instructions: a VALU write of the broadcast register one instruction before
    is a hazard, the same write behind an s_nop 1 or by an LDS read is not, and
    a VALU write of EXEC needs five wait states."""
    import importlib.util
    path = os.path.join(os.path.dirname(ckq.lib_path()), "check_dpp.py")
    spec = importlib.util.spec_from_file_location("check_dpp", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    dpp = "\tv_fmac_f32_dpp v10, v5, v7 row_newbcast:3 row_mask:0xf bank_mask:0xf\n"
    cases = {
        "valu_adjacent": ("\tv_cvt_f32_f16_e32 v5, v9\n" + dpp, 1),
        "valu_two_back": ("\tv_cvt_f32_f16_e32 v5, v9\n\tv_mov_b32_e32 v1, v2\n" + dpp, 1),
        "valu_three_back": ("\tv_cvt_f32_f16_e32 v5, v9\n\tv_mov_b32_e32 v1, v2\n\tv_mov_b32_e32 v3, v2\n" + dpp, 0),
        "valu_then_nop": ("\tv_cvt_f32_f16_e32 v5, v9\n\ts_nop 1\n" + dpp, 0),
        "lds_read": ("\tds_read_b32 v5, v9\n\ts_waitcnt lgkmcnt(0)\n" + dpp, 0),
        "wide_write": ("\tv_pk_mul_lo_u16 v[4:5], v1, v2\n" + dpp, 1),
        "other_register": ("\tv_mov_b32_e32 v6, v9\n" + dpp, 0),
        "valu_exec": ("\tv_cmpx_lt_i32_e32 v1, v2\n\tv_mov_b32_e32 v1, v2\n\tv_mov_b32_e32 v3, v2\n" + dpp, 1),
        "salu_exec": ("\ts_or_b64 exec, exec, s[6:7]\n" + dpp, 0),
    }
    for name, (text, want) in cases.items():
        f = tmp_path / (name + ".s")
        f.write_text(text)
        count, bad = mod.check(str(f))
        assert count == 1 and bad == want, (name, count, bad)
