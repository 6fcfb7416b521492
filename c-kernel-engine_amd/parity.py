"""NumPy / torch front-ends over the C ABI, shaped like the calls the
reference's parity scripts make (ctypes into ck_test_* and the kernel symbols,
e.g. unittest/test_q4_k_q8_k_matvec.py:93-132, unittest/test_parallel_gemv.py:112-170).

Host functions take NumPy arrays and go through the drop-in (host-pointer)
symbols; `dev_*` functions take torch CUDA tensors and go through the
device-resident entry points on torch's current stream."""
import ctypes

import numpy as np

from .api import BLOCK_ELEMS, FMT, STEP, MatmulOp, check, dump_lib, lib, row_bytes

_vp = ctypes.c_void_p


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_vp)


def act_format(wfmt):
    return "q8_0" if wfmt in ("q8_0", "q5_0") else "q8_k"


# ---- host-pointer (drop-in) path ------------------------------------------------

def quantize(x, fmt="q8_k", rows=1):
    """fp32 [rows*k] -> Q8_K / Q8_0 bytes via quantize_batch_*."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.size // rows
    out = np.zeros(rows * row_bytes(fmt, k), dtype=np.uint8)
    fn = lib().quantize_batch_q8_k if fmt == "q8_k" else lib().quantize_batch_q8_0
    fn(_p(x), _p(out), rows, k)
    return out


_GEMV = {"q4_k": "gemv_q4_k_q8_k", "q5_k": "gemv_q5_k_q8_k", "q6_k": "gemv_q6_k_q8_k", "q8_0": "gemv_q8_0_q8_0",
         "q5_0": "gemv_q5_0_q8_0"}
_GEMM_NT = {"q4_k": "gemm_nt_q4_k_q8_k", "q5_k": "gemm_nt_q5_k_q8_k", "q6_k": "gemm_nt_q6_k_q8_k",
            "q8_0": "gemm_nt_q8_0_q8_0", "q5_0": "gemm_nt_q5_0_q8_0"}


def gemv(fmt, W, x_q8, M, K, name=None):
    y = np.zeros(M, dtype=np.float32)
    getattr(lib(), name or _GEMV[fmt])(_p(y), _p(W), _p(x_q8), M, K)
    return y


def gemv_parallel(fmt, W, x_q8, M, K, nth, simd=True, y=None):
    """Union over ith of the thread-split entry point."""
    y = np.zeros(M, dtype=np.float32) if y is None else y
    fn = getattr(lib(), _GEMV[fmt] + ("_parallel_simd" if simd else "_parallel"))
    for ith in range(nth):
        fn(_p(y), _p(W), _p(x_q8), M, K, ith, nth)
    return y


def gemm_nt(fmt, A_q8, B, bias, M, N, K):
    c = np.zeros(M * N, dtype=np.float32)
    getattr(lib(), _GEMM_NT[fmt])(_p(A_q8), _p(B), _p(bias), _p(c), M, N, K)
    return c.reshape(M, N)


def dequant_row(fmt, src, n):
    out = np.zeros(n, dtype=np.float32)
    getattr(lib(), "dequant_%s_row" % fmt)(_p(src), _p(out), n)
    return out


def embedding_forward(fmt, ids, token_count, vocab, table, pos, embed_dim, aligned, context, add_pos, fill=0.0):
    out = np.full(context * aligned, fill, dtype=np.float32)
    getattr(lib(), "embedding_forward_" + fmt)(_p(ids), token_count, vocab, _p(table), _p(pos), _p(out),
                                               embed_dim, aligned, context, add_pos)
    return out.reshape(context, aligned)


def rmsnorm_q8_k_fused(x, gamma, tokens, d_model, aligned=None, eps=1e-6):
    aligned = aligned or d_model
    out = np.zeros(tokens * row_bytes("q8_k", d_model), dtype=np.uint8)
    lib().rmsnorm_q8_k_fused(_p(x), _p(gamma), _p(out), tokens, d_model, aligned, ctypes.c_float(eps))
    return out


CK_DT = {"q4_k": 7, "q6_k": 8, "q8_0": 9, "q8_k": 10, "q5_0": 11}   # the reference's CKDataType values


def fused_mlp_swiglu_prefill_w1w2_quant(x, W1, B1, w1_fmt, W2, B2, w2_fmt, seq_len, embed, aligned_embed,
                                        inter, aligned_inter, output=None, scratch=True):
    """Mirror of the reference symbol; returns the [seq_len, aligned_embed] output
    (or the untouched `output` passed in when the call rejects its arguments)."""
    out = output if output is not None else np.zeros(seq_len * aligned_embed, dtype=np.float32)
    scr = np.zeros(16, dtype=np.uint8) if scratch else None
    lib().fused_mlp_swiglu_prefill_w1w2_quant(_p(x), _p(W1), _p(B1), CK_DT[w1_fmt], _p(W2), _p(B2), CK_DT[w2_fmt],
                                              _p(out), seq_len, embed, aligned_embed, inter, aligned_inter, _p(scr))
    return out.reshape(seq_len, aligned_embed) if out.size == seq_len * aligned_embed else out


def gemv_f32act(fmt, W, x_f32, M, K):
    """gemv_q4_k / gemv_q6_k / gemv_q8_0: fp32 activations, nothing quantized."""
    y = np.zeros(M, dtype=np.float32)
    getattr(lib(), "gemv_" + fmt)(_p(y), _p(W), _p(x_f32), M, K)
    return y


def gemm_nt_f32act(fmt, A_f32, B, bias, M, N, K):
    c = np.zeros(M * N, dtype=np.float32)
    getattr(lib(), "gemm_nt_" + fmt)(_p(A_f32), _p(B), _p(bias), _p(c), M, N, K)
    return c.reshape(M, N)


def gemm_f32act(fmt, W, X_f32, M, N, K):
    """gemm_q4_k / gemm_q6_k / gemm_q8_0: Y[n*M + row]."""
    y = np.zeros(N * M, dtype=np.float32)
    getattr(lib(), "gemm_" + fmt)(_p(y), _p(W), _p(X_f32), M, N, K)
    return y.reshape(N, M)


# ---- device-resident path ---------------------------------------------------------

def _stream():
    import torch
    return _vp(torch.cuda.current_stream().cuda_stream)


def _dp(t):
    return None if t is None else _vp(t.data_ptr())


def to_device(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def dev_quantize(x_t, fmt="q8_k", rows=1):
    import torch
    k = x_t.numel() // rows
    out = torch.empty(rows * row_bytes(fmt, k), dtype=torch.uint8, device=x_t.device)
    fn = lib().ckq_quantize_q8_k_dev if fmt == "q8_k" else lib().ckq_quantize_q8_0_dev
    check(fn(_dp(x_t), _dp(out), rows, k, _stream()), "quantize_dev")
    return out


ACT_F32 = 0x200


def fmt_tag(name):
    """Weight-format tag of a format name; "<fmt>+f32" adds CKQ_ACT_F32 (a sequence entry
    with fp32 activations, no quantization)."""
    return FMT[name[:-4]] | ACT_F32 if name.endswith("+f32") else FMT[name]


def dev_gemm_nt(fmt, A_t, B_t, bias_t, M, N, K, out=None):
    """C[M,N] on the device; M = 1 is the GEMV."""
    import torch
    c = out if out is not None else torch.empty(M * N, dtype=torch.float32, device=B_t.device)
    check(lib().ckq_gemm_nt_dev(fmt_tag(fmt), _dp(A_t), _dp(B_t), _dp(bias_t), _dp(c), M, N, K, N, _stream()),
          "ckq_gemm_nt_dev")
    return c.view(M, N)


def dev_gemv_q8_0_f32(W_t, x_t, M, K):
    import torch
    y = torch.empty(M, dtype=torch.float32, device=W_t.device)
    check(lib().ckq_gemv_q8_0_dev(_dp(y), _dp(W_t), _dp(x_t), M, K, _stream()), "ckq_gemv_q8_0_dev")
    return y


def dev_dequant_rows(fmt, table_t, ids_t, vocab, pos_t, n_valid, n_row, tokens, n_out_rows):
    import torch
    out = torch.full((n_out_rows * n_row,), 7.0, dtype=torch.float32, device=table_t.device)
    check(lib().ckq_dequant_rows_dev(FMT[fmt], _dp(table_t), _dp(ids_t), vocab, _dp(pos_t), _dp(out), n_valid, n_row,
                                     tokens, n_out_rows, _stream()), "ckq_dequant_rows_dev")
    return out.view(n_out_rows, n_row)


def dev_rmsnorm_q8_k_fused(x_t, gamma_t, tokens, d_model, aligned=None, eps=1e-6):
    import torch
    aligned = aligned or d_model
    out = torch.zeros(tokens * row_bytes("q8_k", d_model), dtype=torch.uint8, device=x_t.device)
    check(lib().ckq_rmsnorm_q8_k_fused_dev(_dp(x_t), _dp(gamma_t), _dp(out), tokens, d_model, aligned,
                                           ctypes.c_float(eps), _stream()), "ckq_rmsnorm_q8_k_fused_dev")
    return out


def dev_swiglu_q8_k(gate_t, up_t, rows, k, ld):
    import torch
    out = torch.zeros(rows * row_bytes("q8_k", k), dtype=torch.uint8, device=gate_t.device)
    check(lib().ckq_swiglu_q8_k_dev(_dp(gate_t), _dp(up_t), _dp(out), rows, k, ld, _stream()), "ckq_swiglu_q8_k_dev")
    return out


def dev_gemm_nt_f32act(fmt, A_t, B_t, bias_t, M, N, K, out=None):
    import torch
    c = out if out is not None else torch.empty(M * N, dtype=torch.float32, device=B_t.device)
    check(lib().ckq_gemm_nt_f32act_dev(FMT[fmt], _dp(A_t), _dp(B_t), _dp(bias_t), _dp(c), M, N, K, N, _stream()),
          "ckq_gemm_nt_f32act_dev")
    return c


def dev_subblock_dots(fmt, W_t, x_t, M, K):
    import torch
    per = (K // 16) if fmt == "q6_k" else (K // 32)
    out = torch.zeros(M * per, dtype=torch.int32, device=W_t.device)
    check(dump_lib().ckq_subblock_dots_dev(FMT[fmt], _dp(out), _dp(W_t), _dp(x_t), M, K, _stream()),
          "ckq_subblock_dots_dev")
    return out.view(M, per)


def dev_subblock_dots_tokens(fmt, W_t, X_t, M, K, ntok):
    """Raw integer sub-block dots of every (token, row), from the instantiation of
    the streaming kernel a matmul of this shape and token count runs: [ntok, M, K/sub]."""
    import torch
    per = (K // 16) if fmt == "q6_k" else (K // 32)
    out = torch.zeros(ntok * M * per, dtype=torch.int32, device=W_t.device)
    check(dump_lib().ckq_subblock_dots_tokens_dev(FMT[fmt], _dp(out), _dp(W_t), _dp(X_t), M, K, ntok, _stream()),
          "ckq_subblock_dots_tokens_dev")
    return out.view(ntok, M, per)


def dev_subblock_dots_group(fmt, W_ts, X_ts, rows, K, ntok):
    """The same dump from ONE grouped launch over the problems (W_ts[g], X_ts[g],
    rows[g]): [n, ntok, max(rows), K/sub]; rows beyond rows[g] stay zero."""
    import torch
    n, per, mx = len(W_ts), (K // 16) if fmt == "q6_k" else (K // 32), max(rows)
    out = torch.zeros(n * ntok * mx * per, dtype=torch.int32, device=W_ts[0].device)
    Wp = (_vp * n)(*[w.data_ptr() for w in W_ts])
    Xp = (_vp * n)(*[x.data_ptr() for x in X_ts])
    rp = (ctypes.c_int * n)(*rows)
    check(dump_lib().ckq_subblock_dots_group_dev(FMT[fmt], n, _dp(out), ctypes.cast(Wp, _vp), ctypes.cast(Xp, _vp),
                                            ctypes.cast(rp, _vp), K, ntok, _stream()), "ckq_subblock_dots_group_dev")
    return out.view(n, ntok, mx, per)


def dev_gemm_block_sums(fmt, A_t, B_t, bias_t, M, N, K):
    """The matrix-core GEMM with its integer block sums: (C [M,N], sums [M,N,nblk,per])."""
    import torch
    nblk, per = (K // 32, 1) if fmt == "q8_0" else (K // 256, 1 if fmt == "q6_k" else 2)
    c = torch.empty(M * N, dtype=torch.float32, device=B_t.device)
    sums = torch.zeros(M * N * nblk * per, dtype=torch.int32, device=B_t.device)
    check(dump_lib().ckq_gemm_block_sums_dev(FMT[fmt], _dp(A_t), _dp(B_t), _dp(bias_t), _dp(c), _dp(sums), M, N, K, _stream()),
          "ckq_gemm_block_sums_dev")
    return c.view(M, N), sums.view(M, N, nblk, per)


def dev_matmul_sequence(ops, repeat=1):
    """ops: list of matmul entries (fmt, A_t, B_t, bias_t, C_t, M, N, K[, ldc]) and producer
    entries (step, A_t, B_t or None, C_t, M, K[, ld[, eps]]) with step one of
    "quantize_q8_k", "quantize_q8_0", "rmsnorm_q8_k", "swiglu_q8_k"; enqueued
    back-to-back `repeat` times by one C call (no Python between launches)."""
    arr = (MatmulOp * len(ops))()
    for i, op in enumerate(ops):
        if op[0] in STEP:
            step, A_t, B_t, C_t, M, K = op[:6]
            ld = op[6] if len(op) > 6 else 0
            eps = op[7] if len(op) > 7 else 0.0
            arr[i] = MatmulOp(STEP[step], M, 0, K, ld, A_t.data_ptr(), B_t.data_ptr() if B_t is not None else None,
                              None, C_t.data_ptr(), eps)
        else:
            fmt, A_t, B_t, bias_t, C_t, M, N, K = op[:8]
            ldc = op[8] if len(op) > 8 else N
            arr[i] = MatmulOp(fmt_tag(fmt), M, N, K, ldc, A_t.data_ptr(), B_t.data_ptr(),
                              bias_t.data_ptr() if bias_t is not None else None, C_t.data_ptr(), 0.0)
    check(lib().ckq_matmul_sequence_dev(ctypes.cast(arr, _vp), len(ops), repeat, _stream()), "ckq_matmul_sequence_dev")
