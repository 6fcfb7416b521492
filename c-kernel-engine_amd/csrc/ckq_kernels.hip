/*
 * ckq_kernels.hip - gfx950 kernels of the quantized dequant-dot path and their
 * C launchers.
 *
 *   gemv_kernel<F,...>      weight rows x up to 8 activation rows (decode and
 *                           small-batch prefill); weights are streamed once
 *                           with 128-bit loads, unpacked in registers, dotted
 *                           with v_dot4_i32_i8, reduced with DPP.
 *   quantize_q8_k_kernel    fp32 -> Q8_K, bit-exact with the reference; also SiLU(gate)*up -> Q8_K
 *   quantize_q8_0_kernel    fp32 -> Q8_0, bit-exact with the reference
 *   rmsnorm_q8_k_fused_kernel  RMSNorm -> Q8_K in one pass, bit-exact with the reference's FMA build
 *   dequant_rows_kernel     row dequantizers / quantized embedding lookup, bit-exact
 *   copy_kernel             plain streaming copy (counter calibration)
 *   read_kernel             plain streaming read (launch-floor calibration)
 *
 * wave64 only; every kernel is launched with 256-thread blocks.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "ckq_blocks.h"
#include "ckq_formats.hpp"
#include "ckq_producers.hpp"
#include "ckq_launch.h"
#include "ckq_pure.h"

/* ========================================================================= */
/* GEMV                                                                       */
/* ========================================================================= */

/* Which kernel serves a matmul of `ntok` tokens.  The weight-streaming dot4
 * kernel takes up to eight tokens per pass over the weights; the matrix-core
 * GEMMs read the weights once for any token count but have a floor of 13-19 us
 * (their K loop waits on global->LDS copies of ~1.5 us latency with only two or
 * three stages to cover it).  Measured crossover: one pass always streams;
 * beyond that the streaming kernel stays ahead while (passes x weight bytes,
 * at least 3 MB each) fits the budget - 20 MB, 40 MB for the Q5_K GEMM whose
 * floor is higher.  Examples at 9-16 tokens: Q4_K 4096x4096 (9.4 MB) streams
 * (12 us against 14), 11008x4096 (25 MB) goes to the matrix cores (19 us
 * against 25-28), the Q8_0 LM head 151936x896 likewise (67 us against 89-102);
 * Q8_0 4864x896 streams up to 32 tokens. */
constexpr int CKQ_STREAM_TOKENS = 8;
#include <atomic>
static std::atomic<int> g_gemm_policy{0};      /* 0 automatic, 1 matrix cores above one pass, 2 always stream */

extern "C" void ckq_launch_set_gemm_policy(int policy) { g_gemm_policy.store(policy < 0 || policy > 2 ? 0 : policy); }

/* Q8_0 has its own estimate, fitted to the same kind of measurements after its
 * streaming kernel went to aligned loads (us, weight bytes in MB): streaming
 * 4.8 + passes * MB / 5.0 (MB / 3.6 for rows it must read with 2-byte-aligned
 * loads), matrix cores max(14, 9 + MB / 2.5).  LM head 151936x896 (145 MB):
 * 9-16 tokens stream (63-66 us against 67-69), 17 and more go to the matrix
 * cores (89 against 69); 4864x896 (4.6 MB) streams up to 72 tokens (64 tokens:
 * 11.8 us against 15.3). */
static bool gemm_q80_on_matrix_cores(int ntok, size_t weight_bytes, bool aligned_rows)
{
    const int policy = g_gemm_policy.load(std::memory_order_relaxed);
    if (ntok <= CKQ_STREAM_TOKENS || policy == 2) return false;
    if (policy == 1) return true;
    const float passes = (float)((ntok + CKQ_STREAM_TOKENS - 1) / CKQ_STREAM_TOKENS), mb = (float)weight_bytes * 1e-6f;
    const float t_stream = 4.8f + passes * mb / (aligned_rows ? 5.0f : 3.6f);
    const float t_matrix = fmaxf(14.0f, 9.0f + mb / 2.5f);
    return t_stream > t_matrix;
}

static bool gemm_on_matrix_cores(int ntok, size_t weight_bytes, size_t budget_mb)
{
    const int policy = g_gemm_policy.load(std::memory_order_relaxed);
    if (ntok <= CKQ_STREAM_TOKENS || policy == 2) return false;
    if (policy == 1) return true;
    const size_t passes = (size_t)(ntok + CKQ_STREAM_TOKENS - 1) / CKQ_STREAM_TOKENS;
    const size_t per = weight_bytes > ((size_t)3 << 20) ? weight_bytes : ((size_t)3 << 20);
    return passes * per > (budget_mb << 20);
}

#include "ckq_gemv.hpp"
#include "ckq_gemm_common.hpp"

/* C = bias + partial 0 + partial 1 + ... in that order: the result does not
 * depend on which block finished first.  One thread per output. */
__global__ void __launch_bounds__(256) gemm_splitk_reduce_kernel(float *__restrict__ C, long ldc, const float *__restrict__ part,
                                                                 const float *__restrict__ bias, int M, int N, int splits)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, mn = (size_t)M * (size_t)N;
    if (i >= mn) return;
    const int t = (int)(i / (size_t)N), n = (int)(i % (size_t)N);
    float v = part[i];
    for (int s = 1; s < splits; ++s) v += part[(size_t)s * mn + i];
    C[(size_t)t * ldc + n] = bias ? v + bias[n] : v;
}


static std::recursive_mutex g_split_mu;
std::recursive_mutex &gemm_split_mutex() { return g_split_mu; }

/* Grow-only device scratch per (device, stream, kind); see ckq_gemm_common.hpp.
 * kind 0: partial tiles of a K split; kind 1: weights rewritten for another kernel.
 * When all slots are taken the least recently used one is recycled: the device is
 * synchronised (its stream may no longer exist), its buffer freed.  A destroyed
 * stream whose handle value is given out again finds the old stream's slot: harmless,
 * that stream's work has ended and the buffer is still this device's memory.
 * ckq_launch_release_stream gives a stream's slots back explicitly. */
namespace {
constexpr int WS_SLOTS = 32;
struct WsSlot { hipStream_t s; int kind, dev; void *p; size_t cap; unsigned epoch; };
WsSlot   g_ws[WS_SLOTS];
uint64_t g_ws_key[WS_SLOTS], g_ws_use[WS_SLOTS], g_ws_clock = 0;
uint64_t ws_key(int dev, hipStream_t s, int kind)
{
    /* lossless for user-space handles (below 2^56), 32 devices and four kinds; never 0 */
    return (1ull << 63) | ((uint64_t)(kind & 3) << 61) | ((uint64_t)(dev & 31) << 56) | ((uint64_t)(uintptr_t)s & ((1ull << 56) - 1));
}
}

static int workspace_slot(int kind, hipStream_t s, size_t bytes, WsSlot **out, bool *fresh);

int gemm_workspace(int kind, hipStream_t s, size_t bytes, float **out)
{
    WsSlot *sl = nullptr;
    const int rc = workspace_slot(kind, s, bytes, &sl, nullptr);
    if (rc == 0) *out = (float *)sl->p;
    return rc;
}

static int workspace_slot(int kind, hipStream_t s, size_t bytes, WsSlot **out, bool *fresh)
{
    std::lock_guard<std::recursive_mutex> lock(g_split_mu);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const uint64_t key = ws_key(dev, s, kind);
    int i = ckq_workspace_pick(g_ws_key, g_ws_use, WS_SLOTS, key);
    WsSlot *sl = &g_ws[i];
    if (g_ws_key[i] != key) {
        if (g_ws_key[i] != 0 && sl->p) {                 /* recycle */
            int cur = dev;
            if (sl->dev != cur) (void)hipSetDevice(sl->dev);
            e = hipDeviceSynchronize();
            if (e == hipSuccess) e = hipFree(sl->p);
            if (sl->dev != cur) (void)hipSetDevice(cur);
            if (e != hipSuccess) return (int)e;
        }
        g_ws_key[i] = key;
        *sl = {s, kind, dev, nullptr, 0, 0u};
    }
    g_ws_use[i] = ++g_ws_clock;
    if (fresh) *fresh = sl->cap < bytes;
    if (sl->cap < bytes) {
        if (sl->p) {
            e = hipStreamSynchronize(s);
            if (e != hipSuccess) return (int)e;
            (void)hipFree(sl->p);
            sl->p = nullptr; sl->cap = 0;
        }
        const size_t cap = bytes + bytes / 2;
        e = hipMalloc(&sl->p, cap);
        if (e != hipSuccess) return (int)e;
        sl->cap = cap;
    }
    *out = sl;
    return 0;
}

/* Frees the scratch held for `stream` on the current device (call before the
 * stream is destroyed, after its work has been synchronised). */
extern "C" int ckq_launch_release_stream(void *stream)
{
    std::lock_guard<std::recursive_mutex> lock(g_split_mu);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    for (int i = 0; i < WS_SLOTS; ++i) {
        if (g_ws_key[i] == 0 || g_ws[i].s != (hipStream_t)stream || g_ws[i].dev != dev) continue;
        if (g_ws[i].p) {
            e = hipStreamSynchronize((hipStream_t)stream);
            if (e != hipSuccess) return (int)e;
            (void)hipFree(g_ws[i].p);
        }
        g_ws_key[i] = 0;
        g_ws_use[i] = 0;
        g_ws[i] = {};
    }
    return 0;
}


int gemm_launch_reduce(float *C, long ldc, const float *part, const float *bias, int M, int N, int splits, hipStream_t s)
{
    const size_t mn = (size_t)M * (size_t)N;
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((mn + 255) / 256)), dim3(256), 0, s,
                       C, ldc, part, bias, M, N, splits);
    return (int)hipGetLastError();
}



/* Q5_0 block -> Q8_0 block: the scale is kept, the 32 values become int8
 * q - 16.  One thread per block. */
__global__ void __launch_bounds__(256) q5_0_to_q8_0_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, size_t nblocks)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nblocks) return;
    FmtQ50::Wt w;
    FmtQ50::Off o;
    o.blk = 0;
    FmtQ50::load_w(w, src + i * 22, o);
    FmtQ50::Dec d;
    FmtQ50::decode(d, w, 0);
    uint8_t *out = dst + i * 34;
    *reinterpret_cast<uint16_t *>(out) = (uint16_t)w.d;
#pragma unroll
    for (int k = 0; k < 8; ++k) {             /* 34-byte blocks: 2-byte aligned stores */
        reinterpret_cast<uint16_t *>(out + 2)[2 * k] = (uint16_t)((u32)d.q[k] & 0xffffu);
        reinterpret_cast<uint16_t *>(out + 2)[2 * k + 1] = (uint16_t)((u32)d.q[k] >> 16);
    }
}

static int launch_gemm_q50_via_q80(const void *A, const void *B, const float *bias, float *C,
                                   int M, int N, int K, long ldc, hipStream_t s)
{
    const size_t nblocks = (size_t)N * (size_t)(K / 32);
    std::lock_guard<std::recursive_mutex> lock(g_split_mu);   /* the scratch is shared by launches on this stream */
    float *tmp = nullptr;
    int rc = gemm_workspace(1, s, nblocks * 34, &tmp);
    if (rc) return rc;
    hipLaunchKernelGGL(q5_0_to_q8_0_kernel, dim3((unsigned)((nblocks + 255) / 256)), dim3(256), 0, s,
                       (const uint8_t *)B, (uint8_t *)tmp, nblocks);
    rc = (int)hipGetLastError();
    if (rc) return rc;
    return launch_gemm_q80_mfma(A, tmp, bias, C, M, N, K, ldc, GemmOpts{}, s);
}

static bool weights_dword_aligned(const GemvArgs &a, const GemvGroup &grp)
{
    uintptr_t bits = reinterpret_cast<uintptr_t>(a.W);
    for (int i = 0; i + 1 < grp.n; ++i) bits |= reinterpret_cast<uintptr_t>(grp.W[i]);
    return (bits & 3) == 0;
}

static const GemvGroup k_no_group = {{}, {}, {}, {}, {}, {}, 1};

static int launch_gemv_args(int fmt, GemvArgs &a, const GemvGroup &grp, int K, void *stream, const GemmOpts &opts = GemmOpts{});

/* `subdots`, when non-NULL, selects the dump build of the instantiation the
 * same call would run without it: out[(t * nrows + row) * nsub + i], nothing
 * is written to y. */
extern "C" int ckq_launch_gemv(int fmt, float *y, const void *W, const void *X, const float *bias,
                               int nrows, int K, int ntok, long ldy, int row0, int row1,
                               int32_t *subdots, void *stream)
{
    if ((!y && !subdots) || !W || !X || nrows <= 0 || K <= 0 || ntok <= 0) return CKQ_EINVAL;
    if (row0 < 0) row0 = 0;
    if (row1 > nrows) row1 = nrows;
    if (row0 >= row1) return 0;
    if (subdots && ntok > CKQ_STREAM_TOKENS) return CKQ_EINVAL;
    GemvArgs a = {};
    a.y = y; a.W = (const uint8_t *)W; a.X = (const uint8_t *)X; a.bias = bias; a.sub = subdots;
    a.nrows = nrows; a.ntok = ntok; a.row0 = row0; a.row1 = row1; a.ldy = ldy;
    return launch_gemv_args(fmt, a, k_no_group, K, stream);
}

/* LDS bytes of the staged token tile of a grouped launch against the 64 KB a
 * block may use: MT rows of activations, MT = token count rounded up to the
 * tile sizes launch_mt knows (1, 2, 4, 8); Q8_0 activations are re-laid out to
 * 36 bytes per block. */
static bool group_tile_fits_lds(int fmt, int K, int ntok)
{
    const size_t mt = ntok <= 1 ? 1 : ntok == 2 ? 2 : ntok <= 4 ? 4 : 8;
    size_t bytes;
    switch (fmt) {
    case CKQ_FMT_Q4_K: case CKQ_FMT_Q5_K: case CKQ_FMT_Q6_K: bytes = FmtQ4K::xs_lds_bytes(mt * (size_t)(K / 256) * 292); break;
    case CKQ_FMT_Q8_0: case CKQ_FMT_Q5_0:                     bytes = FmtQ80::xs_lds_bytes(mt * (size_t)(K / 32) * 34); break;
    default: return false;
    }
    return bytes <= 65536;
}

/* `n` (2..CKQ_GROUP_MAX) independent matmuls of one format and input width,
 * each with its own number of rows - the Q/K/V (grouped-query attention makes
 * K and V narrower than Q) or the gate/up projections of a token - as one
 * launch of the streaming kernel: the launches' fixed start-up cost is paid
 * once and the chip holds n times the loads in flight.  Up to eight tokens; a
 * token tile too large for LDS is issued as separate launches.  `subdots`,
 * when non-NULL, runs the dump build of the grouped instantiation instead:
 * out[((g * ntok + t) * max_rows + row) * nsub + i]. */
extern "C" int ckq_launch_gemv_group(int fmt, int n, float *const *y, const void *const *W, const void *const *X,
                                     const float *const *bias, const int *rows, const long *ldys, int K, int ntok,
                                     int32_t *subdots, void *stream)
{
    if (n < 1 || n > CKQ_GROUP_MAX || !W || !X || !rows || K <= 0 || ntok < 1 || ntok > CKQ_STREAM_TOKENS)
        return CKQ_EINVAL;
    if (!subdots && (!y || !ldys)) return CKQ_EINVAL;
    int nrows = 0;                                  /* the grid and the launch shape follow the largest problem */
    for (int i = 0; i < n; ++i) {
        if (rows[i] <= 0) return CKQ_EINVAL;
        if (rows[i] > nrows) nrows = rows[i];
    }
    for (int i = 0; i < n && !subdots; ++i)
        if (ldys[i] < rows[i] || ldys[i] > 0x7fffffff || !y[i]) return CKQ_EINVAL;
    for (int i = 0; i < n; ++i)
        if (!W[i] || !X[i]) return CKQ_EINVAL;
    /* Every grouped kernel stages its token tile in LDS.  A tile that does not
     * fit (the tile is the token count rounded up to 1, 2, 4 or 8 rows of
     * activations) goes out as n separate launches, which stream it instead. */
    if (n == 1 || !group_tile_fits_lds(fmt, K, ntok)) {
        if (subdots) return CKQ_EINVAL;
        for (int i = 0; i < n; ++i) {
            const int rc = ckq_launch_gemv(fmt, y[i], W[i], X[i], bias ? bias[i] : nullptr, rows[i], K, ntok, ldys[i], 0,
                                           rows[i], nullptr, stream);
            if (rc) return rc;
        }
        return 0;
    }
    GemvArgs a = {};
    GemvGroup grp = k_no_group;
    a.y = subdots ? nullptr : y[0]; a.W = (const uint8_t *)W[0]; a.X = (const uint8_t *)X[0];
    a.bias = bias && !subdots ? bias[0] : nullptr; a.sub = subdots;
    a.nrows = nrows; a.ntok = ntok; a.row0 = 0; a.row1 = rows[0]; a.ldy = subdots ? nrows : ldys[0];
    for (int i = 1; i < n; ++i) {
        grp.y[i - 1] = subdots ? nullptr : y[i]; grp.W[i - 1] = (const uint8_t *)W[i]; grp.X[i - 1] = (const uint8_t *)X[i];
        grp.bias[i - 1] = bias && !subdots ? bias[i] : nullptr;
        grp.nrows[i - 1] = rows[i];
        grp.ldy[i - 1] = subdots ? nrows : (int)ldys[i];
    }
    grp.n = n;
    return launch_gemv_args(fmt, a, grp, K, stream);
}

static int launch_gemv_args(int fmt_flags, GemvArgs &a, const GemvGroup &grp, int K, void *stream, const GemmOpts &opts)
{
    int fmt = fmt_flags;
    float *const y = a.y;
    const void *const W = a.W, *const X = a.X;
    const float *const bias = a.bias;
    const int nrows = a.nrows, ntok = a.ntok, row0 = a.row0, row1 = a.row1;
    const long ldy = a.ldy;
    hipStream_t s = (hipStream_t)stream;
    const bool dump = a.sub != nullptr;
    const bool whole = !dump && grp.n == 1 && row0 == 0 && row1 == nrows;   /* what a matrix-core GEMM can take */
    switch (fmt) {
    case CKQ_FMT_Q4_K:
        if (K % 256) return CKQ_ESHAPE;
        if (whole && gemm_on_matrix_cores(ntok, (size_t)nrows * (K / 256) * 144, 20))
            return launch_gemm_q4k_mfma(X, W, bias, y, ntok, nrows, K, ldy, opts, s);
        a.npos = K / 64; a.wrow = (long)(K / 256) * 144; a.xrow = (long)(K / 256) * 292; a.nsub_row = K / 32;
        return ckq_gemv_launch_q4k(a, grp, s);
    case CKQ_FMT_Q5_K:
        if (K % 256) return CKQ_ESHAPE;
        if (whole && gemm_on_matrix_cores(ntok, (size_t)nrows * (K / 256) * 176, 40))
            return launch_gemm_q5k_mfma(X, W, bias, y, ntok, nrows, K, ldy, opts, s);
        a.npos = K / 64; a.wrow = (long)(K / 256) * 176; a.xrow = (long)(K / 256) * 292; a.nsub_row = K / 32;
        return ckq_gemv_launch_q5k(a, grp, s);
    case CKQ_FMT_Q6_K:
        if (K % 256) return CKQ_ESHAPE;
        if (whole && gemm_on_matrix_cores(ntok, (size_t)nrows * (K / 256) * 210, 20))
            return launch_gemm_q6k_mfma(X, W, bias, y, ntok, nrows, K, ldy, opts, s);
        a.npos = K / 64; a.wrow = (long)(K / 256) * 210; a.xrow = (long)(K / 256) * 292; a.nsub_row = K / 16;
        return ckq_gemv_launch_q6k(a, grp, s);
    case CKQ_FMT_Q8_0:
        if (K % 32) return CKQ_ESHAPE;
        if (whole && gemm_q80_on_matrix_cores(ntok, (size_t)nrows * (K / 32) * 34, K % 64 == 0 && weights_dword_aligned(a, grp)))
            return launch_gemm_q80_mfma(X, W, bias, y, ntok, nrows, K, ldy, opts, s);
        a.wrow = (long)(K / 32) * 34; a.xrow = (long)(K / 32) * 34; a.nsub_row = K / 32;
        /* rows of an even number of blocks at dword-aligned addresses: two blocks per position, aligned loads */
        if (K % 64 == 0 && weights_dword_aligned(a, grp)) {
            a.npos = K / 64;
            return ckq_gemv_launch_q80p(a, grp, s);
        }
        a.npos = K / 32;
        return ckq_gemv_launch_q80(a, grp, s);
    case CKQ_FMT_Q5_0:
        if (K % 32) return CKQ_ESHAPE;
        /* prefill: the blocks are rewritten as Q8_0 blocks (same scale, values
         * q - 16: every dot product is unchanged) and go to the Q8_0 GEMM */
        if (whole && gemm_on_matrix_cores(ntok, (size_t)nrows * (K / 32) * 22, 20)) {
            if (opts.scratch) return CKQ_ESCRATCH;       /* the rewritten weights would need an allocation */
            return launch_gemm_q50_via_q80(X, W, bias, y, ntok, nrows, K, ldy, s);
        }
        a.npos = K / 32; a.wrow = (long)(K / 32) * 22; a.xrow = (long)(K / 32) * 34; a.nsub_row = K / 32;
        return ckq_gemv_launch_q50(a, grp, s);
    case CKQ_KERNEL_Q80_F32:
        if (K % 32) return CKQ_ESHAPE;
        if (dump || grp.n > 1) return CKQ_EINVAL;
        a.npos = K / 32; a.wrow = (long)(K / 32) * 34; a.xrow = (long)K * 4; a.nsub_row = K / 32;
        return ckq_gemv_launch_q80_f32(a, grp, s);
    case CKQ_KERNEL_Q4K_F32:
        if (K % 256) return CKQ_ESHAPE;
        if (dump || grp.n > 1) return CKQ_EINVAL;
        a.npos = K / 64; a.wrow = (long)(K / 256) * 144; a.xrow = (long)K * 4; a.nsub_row = K / 64;
        return ckq_gemv_launch_q4k_f32(a, grp, s);
    case CKQ_KERNEL_Q6K_F32:
        if (K % 256) return CKQ_ESHAPE;
        if (dump || grp.n > 1) return CKQ_EINVAL;
        a.npos = K / 64; a.wrow = (long)(K / 256) * 210; a.xrow = (long)K * 4; a.nsub_row = K / 64;
        return ckq_gemv_launch_q6k_f32(a, grp, s);
    default:
        return CKQ_EFORMAT;
    }
}

/* Several weight matrices of one format against the same quantized activations (Q/K/V, gate/up at
 * prefill sizes) as ONE matrix-core launch: the tiles of all matrices share a grid, so the narrow ones
 * (K and V under grouped-query attention) fill the chip together with the wide one instead of each
 * taking a K-split launch of its own, and one launch boundary replaces n.  Every tile is computed
 * exactly as the single-matrix launch without a K split computes it.  CKQ_ENOGROUP: not taken (the
 * streaming kernel would serve these sizes, or the tiles of all matrices together still leave most of
 * the chip idle); the caller then issues the matrices one by one. */
extern "C" int ckq_launch_gemm_group(int fmt, int n, float *const *C, const void *const *B, const void *A,
                                     const float *const *bias, const int *N, const long *ldc, int K, int M, void *stream)
{
    if (n < 2 || n > GEMM_GROUP_MAX || M <= CKQ_STREAM_TOKENS || !A || K <= 0) return CKQ_ENOGROUP;
    GemmGroupIn in = {};
    in.n = n;
    size_t rows = 0;
    bool aligned = true;
    for (int p = 0; p < n; ++p) {
        if (!C[p] || !B[p] || N[p] <= 0 || ldc[p] < N[p]) return CKQ_EINVAL;
        in.B[p] = B[p]; in.bias[p] = bias ? bias[p] : nullptr; in.C[p] = C[p]; in.N[p] = N[p]; in.ldc[p] = ldc[p];
        rows += (size_t)N[p];
        aligned = aligned && ((uintptr_t)B[p] % 4 == 0);
    }
    hipStream_t s = (hipStream_t)stream;
    switch (fmt) {
    case CKQ_FMT_Q4_K:
        if (K % 256) return CKQ_ESHAPE;
        if (!gemm_on_matrix_cores(M, rows * (K / 256) * 144, 20)) return CKQ_ENOGROUP;
        return launch_gemm_q4k_mfma_group(A, in, M, K, s);
    case CKQ_FMT_Q5_K:
        if (K % 256) return CKQ_ESHAPE;
        if (!gemm_on_matrix_cores(M, rows * (K / 256) * 176, 40)) return CKQ_ENOGROUP;
        return launch_gemm_q5k_mfma_group(A, in, M, K, s);
    case CKQ_FMT_Q6_K:
        if (K % 256) return CKQ_ESHAPE;
        if (!gemm_on_matrix_cores(M, rows * (K / 256) * 210, 20)) return CKQ_ENOGROUP;
        return launch_gemm_q6k_mfma_group(A, in, M, K, s);
    case CKQ_FMT_Q8_0:
        if (K % 32) return CKQ_ESHAPE;
        if (!gemm_q80_on_matrix_cores(M, rows * (K / 32) * 34, K % 64 == 0 && aligned)) return CKQ_ENOGROUP;
        return launch_gemm_q80_mfma_group(A, in, M, K, s);
    default:
        return CKQ_ENOGROUP;
    }
}

/* ---- the entry point that allocates nothing ---------------------------------
 * Scratch for the partial tiles of a K-split GEMM, held in the code object:
 * every device the library runs on holds its own copy, at its own address,
 * until the process ends.  Host code never uses the array's name as an
 * address: the per-device address comes from hipGetSymbolAddress, once per
 * device, with that device current.  The array keeps the last call's
 * contents; nothing in it has to start at zero (the split kernel writes every
 * partial entry the reduction reads).  Calls that overlap on one GPU race. */
static __device__ __align__(256) unsigned char scratch[CKQ_NOALLOC_SCRATCH_BYTES];
constexpr int CKQ_MAX_DEVICES = 64;
static std::atomic<void *> g_scratch_ptr[CKQ_MAX_DEVICES];

static int noalloc_scratch(void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= CKQ_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return 0;
}

extern "C" int ckq_launch_noalloc_setup(void)
{
    void *p;
    return noalloc_scratch(&p);
}

extern "C" int ckq_launch_gemv_noalloc(int fmt, float *y, const void *W, const void *X, const float *bias,
                                       int nrows, int K, int ntok, long ldy, void *stream)
{
    if (fmt != CKQ_FMT_Q4_K && fmt != CKQ_FMT_Q5_K && fmt != CKQ_FMT_Q6_K && fmt != CKQ_FMT_Q8_0) return CKQ_EFORMAT;
    if (!y || !W || !X || nrows <= 0 || K <= 0 || ntok <= 0 || ldy < nrows) return CKQ_EINVAL;
    void *p = nullptr;
    {
        /* The scratch address of this device is normally resolved by ckq_init().  Resolving it
         * here, on a first call, may load the code object, which is not legal while the stream
         * is being captured: such a call is refused instead. */
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < CKQ_MAX_DEVICES &&
            !g_scratch_ptr[dev].load(std::memory_order_acquire)) {
            hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing((hipStream_t)stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone)
                return (int)hipErrorStreamCaptureUnsupported;
            (void)hipGetLastError();
        }
    }
    const int rc = noalloc_scratch(&p);
    if (rc) return rc;
    GemvArgs a = {};
    a.y = y; a.W = (const uint8_t *)W; a.X = (const uint8_t *)X; a.bias = bias; a.sub = nullptr;
    a.nrows = nrows; a.ntok = ntok; a.row0 = 0; a.row1 = nrows; a.ldy = ldy;
    return launch_gemv_args(fmt, a, k_no_group, K, stream, GemmOpts{nullptr, (float *)p, CKQ_NOALLOC_SCRATCH_BYTES});
}

/* The matrix-core GEMM of `fmt`, whatever the token count, with its integer
 * block sums stored next to the result: sums[((t * N + n) * nblk + b) * per + i],
 * nblk = K / 256 and per = 2 (I1, I2) for Q4_K and Q5_K, per = 1 (I) for Q6_K,
 * nblk = K / 32 and per = 1 (the block dot) for Q8_0.  For the exactness tests. */
extern "C" int ckq_launch_gemm_block_sums(int fmt, const void *A, const void *B, const float *bias, float *C, int32_t *sums,
                                          int M, int N, int K, long ldc, void *stream)
{
    if (!A || !B || !C || !sums || M <= 0 || N <= 0 || K <= 0 || ldc < N) return CKQ_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    switch (fmt) {
    case CKQ_FMT_Q4_K: return K % 256 ? CKQ_ESHAPE : launch_gemm_q4k_mfma(A, B, bias, C, M, N, K, ldc, GemmOpts{sums, nullptr, 0}, s);
    case CKQ_FMT_Q5_K: return K % 256 ? CKQ_ESHAPE : launch_gemm_q5k_mfma(A, B, bias, C, M, N, K, ldc, GemmOpts{sums, nullptr, 0}, s);
    case CKQ_FMT_Q6_K: return K % 256 ? CKQ_ESHAPE : launch_gemm_q6k_mfma(A, B, bias, C, M, N, K, ldc, GemmOpts{sums, nullptr, 0}, s);
    case CKQ_FMT_Q8_0: return K % 32 ? CKQ_ESHAPE : launch_gemm_q80_mfma(A, B, bias, C, M, N, K, ldc, GemmOpts{sums, nullptr, 0}, s);
    default: return CKQ_EFORMAT;
    }
}

/* ========================================================================= */
/* Activation quantizers                                                      */
/* ========================================================================= */

/* fp32 -> Q8_K, one wave per 256-element block, lane l owns elements 4l..4l+3
 * (q8k_quantize_block holds the reference's rules).  SWIGLU: the quantizer's
 * input is SiLU(x) * up instead of x.  Rows of the input are ldx floats apart,
 * bpr blocks of 256 per row. */
template <bool SWIGLU>
__global__ void __launch_bounds__(256) quantize_q8_k_kernel(const float *__restrict__ x, const float *__restrict__ up,
                                                            uint8_t *__restrict__ y, long nblocks, int bpr, long ldx)
{
    const long blk = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= nblocks) return;
    pro_quantize_block<SWIGLU>(x, up, y, blk, bpr, ldx, threadIdx.x & 63);
}

/*
 * fp32 -> Q8_0, eight lanes per 32-element block (reference:
 * gemm_kernels_q8_0.c:70-146).  d = amax/127 stored as fp16 (RNE);
 * id = amax ? 127/amax : 0; q = RNE(x*id) saturated.
 */
__global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *__restrict__ x, uint8_t *__restrict__ y,
                                                            long nblocks)
{
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long blk = t >> 3;
    const int  j = (int)(t & 7);
    const bool live = blk < nblocks;
    const long b = live ? blk : nblocks - 1;
    const float4 v = reinterpret_cast<const float4 *>(x + b * 32)[j];
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float d  = amax / 127.0f;
    const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
    int q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = rne_sat_i8(__fmul_rn(e[i], id));
    if (!live) return;
    uint8_t *out = y + b * 34;
    uint16_t *o16 = reinterpret_cast<uint16_t *>(out + 2 + 4 * j);   /* 2-byte aligned */
    o16[0] = (uint16_t)((q[0] & 0xff) | ((q[1] & 0xff) << 8));
    o16[1] = (uint16_t)((q[2] & 0xff) | ((q[3] & 0xff) << 8));
    if (j == 0) *reinterpret_cast<uint16_t *>(out) = __builtin_bit_cast(uint16_t, (_Float16)d);
}

extern "C" int ckq_launch_quantize_q8_k(const float *x, void *y, int rows, int k, void *stream)
{
    if (!x || !y || rows <= 0 || k <= 0) return CKQ_EINVAL;
    if (k % 256) return CKQ_ESHAPE;
    const long nblocks = (long)rows * (k / 256);
    hipLaunchKernelGGL(quantize_q8_k_kernel<false>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       x, (const float *)nullptr, (uint8_t *)y, nblocks, k / 256, (long)k);
    return (int)hipGetLastError();
}

/* y[row] = Q8_K(SiLU(gate[row]) * up[row]), rows of gate and up ld floats apart. */
extern "C" int ckq_launch_swiglu_q8_k(const float *gate, const float *up, void *y, int rows, int k, long ld, void *stream)
{
    if (!gate || !up || !y || rows <= 0 || k <= 0 || ld < k) return CKQ_EINVAL;
    if (k % 256 || ld % 4 || ((uintptr_t)gate | (uintptr_t)up) % 16) return CKQ_ESHAPE;
    const long nblocks = (long)rows * (k / 256);
    hipLaunchKernelGGL(quantize_q8_k_kernel<true>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       gate, up, (uint8_t *)y, nblocks, k / 256, ld);
    return (int)hipGetLastError();
}

extern "C" int ckq_launch_quantize_q8_0(const float *x, void *y, int rows, int k, void *stream)
{
    if (!x || !y || rows <= 0 || k <= 0) return CKQ_EINVAL;
    if (k % 32) return CKQ_ESHAPE;
    const long nblocks = (long)rows * (k / 32);
    hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((unsigned)((nblocks * 8 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, x, (uint8_t *)y, nblocks);
    return (int)hipGetLastError();
}

/*
 * Fused producer RMSNorm -> Q8_K, one block of sixteen waves per token (the
 * arithmetic is rms_row's, ckq_producers.hpp): up to D = 4096 every 256-block of
 * the row has a wave of its own.
 */
constexpr int RMS_WAVES = 16;
__global__ void __launch_bounds__(64 * RMS_WAVES) rmsnorm_q8_k_fused_kernel(const float *__restrict__ input,
                                                                 const float *__restrict__ gamma,
                                                                 uint8_t *__restrict__ y, int d_model, long in_stride,
                                                                 float eps)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    rms_row<RMS_WAVES, 1>(input + (size_t)blockIdx.x * in_stride, gamma, y + (size_t)blockIdx.x * (d_model / 256) * 292,
                          d_model, eps, reinterpret_cast<float *>(smem));
}

extern "C" int ckq_launch_rmsnorm_q8_k_fused(const float *input, const float *gamma, void *y, int tokens, int d_model,
                                             int aligned_embed_dim, float eps, void *stream)
{
    if (!input || !gamma || !y || tokens <= 0 || d_model <= 0 || aligned_embed_dim < d_model) return CKQ_EINVAL;
    if (d_model % 256 || aligned_embed_dim % 4) return CKQ_ESHAPE;
    const size_t lds = (size_t)d_model * 4 + 32;
    if (lds > 160 * 1024) return CKQ_ESHAPE;               /* the row is staged in LDS */
    if (lds > 64 * 1024) {
        /* more than 64 KB of dynamic LDS is an opt-in per function and per device: set on every
         * such call for the device that is current (rows this long are rare; the call is cheap) */
        hipError_t e = hipFuncSetAttribute((const void *)rmsnorm_q8_k_fused_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(rmsnorm_q8_k_fused_kernel, dim3((unsigned)tokens), dim3(64 * RMS_WAVES), lds, (hipStream_t)stream,
                       input, gamma, (uint8_t *)y, d_model, (long)aligned_embed_dim, eps);
    return (int)hipGetLastError();
}

/* ========================================================================= */
/* Row dequantizers and quantized embedding lookup                            */
/* ========================================================================= */

/* Four consecutive elements e..e+3 (e % 4 == 0) of a quantized row, with the
 * reference's operation order; products and differences are rounded one by one
 * (reference: dequant_kernels.c:276-296 Q8_0, :336-385 Q4_K, :396-430 Q6_K). */
template <int FMT>
__device__ __forceinline__ float4 dequant4(const uint8_t *row, u32 e)
{
#pragma clang fp contract(off)
    float v[4];
    if (FMT == CKQ_FMT_Q8_0) {
        const uint8_t *blk = row + (e >> 5) * 34u;
        const float d = h2f(ld2(blk));
        const u32 q = ld2(blk + 2 + (e & 31)) | (ld2(blk + 4 + (e & 31)) << 16);
        for (int i = 0; i < 4; ++i) v[i] = d * (float)sbyte(q, i);
    } else if (FMT == CKQ_FMT_Q4_K) {
        const uint8_t *blk = row + (e >> 8) * 144u;
        const u32 w = e & 255, j = w >> 5, l = w & 31;       /* sub-block j, element l of it */
        const u32 hdr0 = ld4<4>(blk);
        u32 sc2, mn2;
        k4_scale_pair(ld4<4>(blk + 4), ld4<4>(blk + 8), ld4<4>(blk + 12), (int)(j >> 1), &sc2, &mn2);
        const u32 sc = (sc2 >> (8 * (j & 1))) & 0xff, mn = (mn2 >> (8 * (j & 1))) & 0xff;
        const float dj = h2f(hdr0 & 0xffff) * (float)sc, mj = h2f(hdr0 >> 16) * (float)mn;
        const u32 qs = ld4<4>(blk + 16 + 32 * (j >> 1) + l);
        const u32 nib = (j & 1) ? (qs >> 4) & 0x0f0f0f0fu : qs & 0x0f0f0f0fu;
        for (int i = 0; i < 4; ++i) v[i] = dj * (float)((nib >> (8 * i)) & 0xff) - mj;
    } else { /* CKQ_FMT_Q6_K */
        const uint8_t *blk = row + (e >> 8) * 210u;
        const u32 w = e & 255, n = w >> 7, r = (w >> 5) & 3, l = w & 31;   /* half n, run r, element l */
        const uint8_t *ql = blk + 64 * n + l + 32 * (r & 1);
        const uint8_t *qh = blk + 128 + 32 * n + l;
        const u32 lo = ld2(ql) | (ld2(ql + 2) << 16), hi = ld2(qh) | (ld2(qh + 2) << 16);
        const u32 q4 = (r >> 1) ? (lo >> 4) & 0x0f0f0f0fu : lo & 0x0f0f0f0fu;
        const u32 q2 = (hi >> (2 * r)) & 0x03030303u;
        const u32 q = q4 | (q2 << 4);
        const float d = h2f(ld2(blk + 208));
        const float ds = d * (float)(int8_t)blk[192 + 8 * n + 2 * r + (l >> 4)];
        for (int i = 0; i < 4; ++i) v[i] = ds * (float)((int)((q >> (8 * i)) & 0xff) - 32);
    }
    return make_float4(v[0], v[1], v[2], v[3]);
}

/*
 * out[t][0..n_row) for t < n_out_rows: rows t < tokens hold the dequantized
 * source row (ids ? clamp(ids[t]) : t), plus pos[t] where asked, zero from
 * n_valid on; rows from `tokens` on are zero (reference:
 * src/kernels/embedding_kernels.c:76-196).
 */
template <int FMT>
__global__ void __launch_bounds__(256) dequant_rows_kernel(const uint8_t *__restrict__ table, const int32_t *__restrict__ ids,
                                                           int vocab, const float *__restrict__ pos, float *__restrict__ out,
                                                           int n_valid, int n_row, long row_bytes, int tokens, int col_blocks)
{
    /* the output row rides in blockIdx.x with the column block (gridDim.y stops at 65 535 rows) */
    const int t = (int)(blockIdx.x / (u32)col_blocks);
    const u32 e = 4u * ((blockIdx.x % (u32)col_blocks) * 256u + threadIdx.x);
    if (e >= (u32)n_row) return;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t < tokens) {
        long src = t;
        if (ids) {
            const int id = ids[t];
            src = (id < 0 || id >= vocab) ? 0 : id;
        }
        v = dequant4<FMT>(table + src * row_bytes, e);
        if (pos) {
            const float4 p = *reinterpret_cast<const float4 *>(pos + (size_t)t * n_row + e);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        if (e + 0 >= (u32)n_valid) v.x = 0.f;
        if (e + 1 >= (u32)n_valid) v.y = 0.f;
        if (e + 2 >= (u32)n_valid) v.z = 0.f;
        if (e + 3 >= (u32)n_valid) v.w = 0.f;
    }
    *reinterpret_cast<float4 *>(out + (size_t)t * n_row + e) = v;
}

extern "C" int ckq_launch_dequant_rows(int fmt, const void *table, const int32_t *ids, int vocab, const float *pos,
                                       float *out, int n_valid, int n_row, int tokens, int n_out_rows, void *stream)
{
    if (!table || !out || n_row <= 0 || n_out_rows <= 0 || tokens < 0 || n_valid < 0) return CKQ_EINVAL;
    if (fmt != CKQ_FMT_Q4_K && fmt != CKQ_FMT_Q6_K && fmt != CKQ_FMT_Q8_0) return CKQ_EFORMAT;
    if (n_row % (fmt == CKQ_FMT_Q8_0 ? 32 : 256)) return CKQ_ESHAPE;
    if (tokens > n_out_rows) tokens = n_out_rows;
    if (n_valid > n_row) n_valid = n_row;
    const long rb = (long)ckq_row_bytes(fmt, n_row);
    const int col_blocks = (n_row / 4 + 255) / 256;
    if ((long long)col_blocks * n_out_rows > 0x7fffffffll) return CKQ_ESHAPE;
    const dim3 grid((unsigned)((long long)col_blocks * n_out_rows)), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (fmt) {
    case CKQ_FMT_Q4_K:
        hipLaunchKernelGGL(dequant_rows_kernel<CKQ_FMT_Q4_K>, grid, block, 0, s, (const uint8_t *)table, ids, vocab, pos, out, n_valid, n_row, rb, tokens, col_blocks);
        break;
    case CKQ_FMT_Q6_K:
        hipLaunchKernelGGL(dequant_rows_kernel<CKQ_FMT_Q6_K>, grid, block, 0, s, (const uint8_t *)table, ids, vocab, pos, out, n_valid, n_row, rb, tokens, col_blocks);
        break;
    default:
        hipLaunchKernelGGL(dequant_rows_kernel<CKQ_FMT_Q8_0>, grid, block, 0, s, (const uint8_t *)table, ids, vocab, pos, out, n_valid, n_row, rb, tokens, col_blocks);
        break;
    }
    return (int)hipGetLastError();
}

/* ========================================================================= */
/* Streaming copy                                                             */
/* ========================================================================= */
__global__ void __launch_bounds__(256) copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

/* Reads `n16` 16-byte units and keeps nothing: what one launch costs when it
 * only has to pull that many bytes out of HBM (the floor for a GEMV whose
 * weights are that large). */
typedef unsigned ckq_v4u __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) read_kernel(const ckq_v4u *__restrict__ src, size_t n16, unsigned *sink)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n16) return;
    const ckq_v4u v = __builtin_nontemporal_load(src + i);
    if ((v[0] ^ v[1] ^ v[2] ^ v[3]) == 0x9e3779b9u && v[0] == 0x7f4a7c15u) *sink = v[0];   /* never true in practice */
}

/* The same read as a tuned streaming kernel: a grid sized to what the chip
 * holds at once (`blocks` blocks of 256 threads), every lane keeping U
 * independent 16-byte loads in flight per trip and striding through the buffer,
 * so that neither block dispatch nor a one-load-per-lane dependency limits the
 * rate.  The fastest (blocks, U) the benchmark finds is the launch floor it
 * prices the GEMV against. */
template <int U>
__global__ void __launch_bounds__(256) read_stream_kernel(const ckq_v4u *__restrict__ src, size_t n16, unsigned *sink)
{
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    ckq_v4u acc = {0u, 0u, 0u, 0u};
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        ckq_v4u v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u];
    }
    for (; i < n16; i += stride) acc ^= src[i];
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && acc[0] == 0x7f4a7c15u) *sink = acc[0];   /* never true in practice */
}

extern "C" int ckq_launch_read_tuned(const void *src, size_t bytes, void *sink, int blocks, int unroll, void *stream)
{
    if (!src || !sink || bytes < 16 || blocks <= 0) return CKQ_EINVAL;
    const size_t n16 = bytes / 16;
    const dim3 grid((unsigned)blocks), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (unroll) {
    case 1: hipLaunchKernelGGL(read_stream_kernel<1>, grid, block, 0, s, (const ckq_v4u *)src, n16, (unsigned *)sink); break;
    case 2: hipLaunchKernelGGL(read_stream_kernel<2>, grid, block, 0, s, (const ckq_v4u *)src, n16, (unsigned *)sink); break;
    case 4: hipLaunchKernelGGL(read_stream_kernel<4>, grid, block, 0, s, (const ckq_v4u *)src, n16, (unsigned *)sink); break;
    case 8: hipLaunchKernelGGL(read_stream_kernel<8>, grid, block, 0, s, (const ckq_v4u *)src, n16, (unsigned *)sink); break;
    default: return CKQ_EINVAL;
    }
    return (int)hipGetLastError();
}

extern "C" int ckq_launch_read(const void *src, size_t bytes, void *sink, void *stream)
{
    if (!src || !sink || bytes < 16) return CKQ_EINVAL;
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(read_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const ckq_v4u *)src, n16, (unsigned *)sink);
    return (int)hipGetLastError();
}

extern "C" int ckq_launch_copy(void *dst, const void *src, size_t bytes, void *stream)
{
    if (!dst || !src || bytes == 0 || (bytes & 15)) return CKQ_EINVAL;
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (uint4 *)dst, (const uint4 *)src, n16);
    return (int)hipGetLastError();
}
