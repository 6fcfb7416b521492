"""ckq-hip: MI355X (gfx950) implementation of C-Kernel-Engine's quantized
dequant-dot matmul path, driven through ctypes like the reference's own parity
scripts (reference: unittest/lib_loader.py:10-23, unittest/test_q4_k_q8_k_matvec.py).

The directory name is not a Python identifier; import it with
``importlib.import_module("c-kernel-engine_amd")``.

Nothing here computes: every function forwards to libckernel_quant_hip.so and
raises if that library is missing.
"""
from .api import (  # noqa: F401
    BLOCK_BYTES,
    BLOCK_ELEMS,
    FMT,
    CkqError,
    build,
    declared_symbols,
    dump_lib,
    dump_lib_path,
    lib,
    lib_path,
    row_bytes,
    synth_lib,
)
from . import api, parity  # noqa: F401
