/*
 * ckq_gemm_q80.hip - prefill GEMM, Q8_0 weights x Q8_0 activations, on the
 * gfx950 int8 matrix cores.
 *
 *   C[t][n] = sum_j (dw(n,j) * dx(t,j)) * (float) S(t,n,j)   (+ bias[n])
 *   S = sum_{k in 32-block j} w8(n,k) * x8(t,k)                          (exact int32)
 * which is the reference's batched routine (gemm_batch_int8.c:87-120: one
 * integer sum and one product of the two fp16 scales per 32-block).
 *
 * Mapping to the hardware
 * - v_mfma_i32_32x32x32_i8: K = 32 is exactly one Q8_0 block, and both operands
 *   are int8 already, so nothing is unpacked.  Every instruction starts from a
 *   zero accumulator and its 16 outputs per lane are scaled and added into the
 *   fp32 accumulators: three VALU operations per output per block (convert,
 *   product with the token's scale, fused multiply-add with the row's), which is what bounds the kernel; the
 *   matrix pipe is mostly idle and two blocks share a CU to keep the VALU fed.
 * - The weights are the A operand and the tokens the B operand, so a lane holds
 *   ONE token and 16 weight rows of the 32x32 result: the token's scale is one
 *   4-byte LDS read per instruction; of the 16 row scales a lane fetches only the
 *   one of output (lane & 15) - one 4-byte read per block - and the multiply-add
 *   of output r takes lane r of the 16-lane row as its factor (fmac_row_lane).
 * - Operands reach LDS by global->LDS loads: the 32 quants of a block as two
 *   16-byte chunks (block starts are only 2-byte aligned in memory; the loads
 *   accept that), the fp16 scales as 2-byte loads, which land zero-extended in
 *   one dword per lane: arrays [row][block] and [token][block] (four adjacent lanes fetch the four scales of one
 *   136-byte run, so an instruction touches 16 runs instead of 64 rows' worth of cache lines).  Quant chunks
 *   of a row are XOR-swizzled by the row number (rows are 128 bytes apart).
 * - K advances 128 (four blocks) per iteration, two LDS stages of 27 KB, two
 *   blocks per CU (one hides the other's fetch).  The block's waves exchange
 *   data only through those copies: a wait for them and a bare barrier end
 *   an iteration.
 *
 * Block = 4 waves = 64 tokens x 128 weight rows; wave w owns rows 32w..32w+31.
 */
#include "ckq_gemm_common.hpp"
#include <type_traits>

constexpr int GEMM8_BM = 64, GEMM8_BN = 128, GEMM8_KB = 4;   /* tokens, rows, 32-blocks per iteration */

struct Gemm8Stage {
    uint8_t  wq[GEMM8_BN * GEMM8_KB * 32];   /* row r: 8 chunks of 16 B, chunk c in slot c ^ (r & 7) */
    uint8_t  xq[GEMM8_BM * GEMM8_KB * 32];   /* token t likewise */
    u32      wd[GEMM8_KB * GEMM8_BN];        /* fp16 scales zero-extended, [row][block] */
    u32      xd[GEMM8_KB * GEMM8_BM];        /* fp16 scales zero-extended, [token][block] */
};

template <bool DUMP>
__global__ void __launch_bounds__(256, 2) gemm_q80_mfma_kernel(GemmArgs a)
{
    constexpr int BM = GEMM8_BM, BN = GEMM8_BN, KB = GEMM8_KB, NST = 2;
    __shared__ __attribute__((aligned(16))) Gemm8Stage stage[NST];

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int col = lane & 31, half = lane >> 5;
    const int dw_row = mfma32_row_of_lane(lane);      /* row (of the wave's 32) of this lane's output lane & 15 */

    /* token tiles fastest inside an XCD, so each XCD's L2 sees a weight tile once */
    const GemmWork work = gemm_work(a, (a.nb + KB - 1) / KB);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * BN;
    const int nblk = a.nb;                                  /* 32-blocks per row */
    const u32 stride = (u32)nblk * 34u;                     /* bytes per weight row and per activation row */
    const int it0 = work.k0, niter = work.k1;               /* this block runs iterations [it0, niter) */
    const uint8_t *wbase = work.B + (size_t)n0 * stride;       /* uniform */
    const uint8_t *xbase = a.A + (size_t)t0 * stride;       /* uniform */

    /* Copy roles per iteration: weight quants 128 rows x 8 chunks = 16 wave
     * instructions (four per wave), activation quants 8 (two per wave), weight
     * scales 4 blocks x 128 rows = 8 two-byte instructions (two per wave),
     * activation scales 4 (one per wave).  A lane's source offset is fixed up to
     * the iteration's 136-byte advance, except in the last iteration of a K that
     * is not a multiple of 128, where the missing blocks re-read block 0 of the
     * iteration (their products are never used). */
    constexpr int NWQ = 4, NXQ = 2, NWD = 2, NXD = 1, NCOPY = NWQ + NXQ + NWD + NXD;
    u32 wq_g[NWQ], xq_g[NXQ], wd_g[NWD], xd_g[NXD];
    u32 wq_blk[NWQ], xq_blk[NXQ], wd_blk[NWD], xd_blk[NXD];   /* which block of the iteration a copy belongs to */
#pragma unroll
    for (int i = 0; i < NWQ; ++i) {
        const int chunk = (wave + 4 * i) * 64 + lane, row = chunk >> 3, c = (chunk & 7) ^ (row & 7);
        wq_blk[i] = (u32)(c >> 1);
        wq_g[i] = (u32)min(row, work.N - 1 - n0) * stride + 2u + 16u * (u32)(c & 1);
    }
#pragma unroll
    for (int i = 0; i < NXQ; ++i) {
        const int chunk = (wave + 4 * i) * 64 + lane, tok = chunk >> 3, c = (chunk & 7) ^ (tok & 7);
        xq_blk[i] = (u32)(c >> 1);
        xq_g[i] = (u32)min(tok, a.M - 1 - t0) * stride + 2u + 16u * (u32)(c & 1);
    }
#pragma unroll
    for (int i = 0; i < NWD; ++i) {
        const int e = (wave + 4 * i) * 64 + lane;            /* [row][block] entry: the four scales of a row come from one 136-byte run */
        wd_blk[i] = (u32)(e & 3);
        wd_g[i] = (u32)min(e >> 2, work.N - 1 - n0) * stride;
    }
    {
        const int e = wave * 64 + lane;                      /* [token][block] entry */
        xd_blk[0] = (u32)(e & 3);
        xd_g[0] = (u32)min(e >> 2, a.M - 1 - t0) * stride;
    }

    /* the copies address their source as buffer (uniform base in SGPRs) + per-lane
     * 32-bit offset + uniform K offset */
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_k = 0;
    int cp_buf = 0, cp_valid = KB;
    auto copy_begin = [&](int it, int buf) {
        cp_k = it * (KB * 34);
        cp_valid = min(KB, nblk - it * KB);
        cp_buf = buf;
    };
    /* uniform base + one 32-bit lane offset per copy */
    auto blk_ofs = [&](u32 j) { return ((int)j < cp_valid ? j : 0u) * 34u; };
    auto copy_one = [&](int i) {
        if (i < NWQ)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(stage[cp_buf].wq + 1024 * (wave + 4 * i)), 16,
                                                     (int)(wq_g[i] + blk_ofs(wq_blk[i])), cp_k, 0, 0);
        else if (i < NWQ + NXQ)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].xq + 1024 * (wave + 4 * (i - NWQ))), 16,
                                                     (int)(xq_g[i - NWQ] + blk_ofs(xq_blk[i - NWQ])), cp_k, 0, 0);
        else if (i < NWQ + NXQ + NWD)   /* 2-byte loads land zero-extended, one dword per lane */
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(stage[cp_buf].wd + 64 * (wave + 4 * (i - NWQ - NXQ))), 2,
                                                     (int)(wd_g[i - NWQ - NXQ] + blk_ofs(wd_blk[i - NWQ - NXQ])), cp_k, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].xd + 64 * wave), 2,
                                                     (int)(xd_g[0] + blk_ofs(xd_blk[0])), cp_k, 0, 0);
    };

    /* read-side offsets of this lane */
    const int row_l = 32 * wave + col;
    u32 bofs[KB], aofs[KB];
#pragma unroll
    for (int j = 0; j < KB; ++j) {
        bofs[j] = (u32)row_l * 128u + 16u * (u32)((2 * j + half) ^ (row_l & 7));
        aofs[j] = (u32)col * 128u + 16u * (u32)((2 * j + half) ^ (col & 7));   /* token col + 32 ts: same low bits */
    }

    ckq_v16f acc[2];
#pragma unroll
    for (int ts = 0; ts < 2; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ts][r] = 0.0f;

#pragma unroll
    for (int p = 0; p < NST - 1; ++p) {
        copy_begin(min(it0 + p, niter - 1), p);
#pragma unroll
        for (int i = 0; i < NCOPY; ++i) copy_one(i);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);                    /* vmcnt(0): the first stage has landed */
    __builtin_amdgcn_s_barrier();

    auto lds16 = [&](const void *p) { return *reinterpret_cast<const ckq_v4i *>(p); };
    const ckq_v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    /* One iteration (KB blocks); the stage it reads is a compile-time constant
     * (the loop below is unrolled over the two stages): LDS addresses are
     * per-lane registers set up once plus immediates. */
    auto kstep = [&](int it, auto curc) {
        constexpr int cur = decltype(curc)::value;
        const Gemm8Stage &st = stage[cur];
        const int valid = min(KB, nblk - it * KB);
        /* Operands of block j (read one block ahead of their use, through the
         * integer vector types only): the row's quants, the four 16-byte groups
         * of row scales, and per token group the token's quants and scale. */
        ckq_v4i wq[2], xq[2][2];
        u32 dwh[2], dxh[2][2];     /* dwh: the scale of the row of output (lane & 15), one per lane */
        auto read_block = [&](int j) {
            wq[j & 1] = lds16(st.wq + bofs[j]);
            dwh[j & 1] = st.wd[(32 * wave + dw_row) * KB + j];
#pragma unroll
            for (int ts = 0; ts < 2; ++ts) {
                xq[j & 1][ts] = lds16(st.xq + aofs[j] + 32 * 128 * ts);
                dxh[j & 1][ts] = st.xd[(32 * ts + col) * KB + j];
            }
        };
        read_block(0);
        copy_begin(min(it + 1, niter - 1), cur ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        /* Eight slots (block j, token group ts).  The MFMA of slot k+1 is issued
         * before the 16 outputs of slot k are scaled and added, so the matrix
         * pipe works under the VALU; rows of the result = weight rows, columns
         * = tokens. */
        ckq_v16i d[2];
        if (0 < valid) d[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wq[0], xq[0][0], zero16, 0, 0, 0);
#pragma unroll
        for (int k = 0; k < 2 * KB; ++k) {
            const int j = k >> 1, ts = k & 1, jn = (k + 1) >> 1, tn = (k + 1) & 1;
            if (ts == 0 && j + 1 < KB) read_block(j + 1);
            if (k + 1 < 2 * KB && jn < valid)
                d[(k + 1) & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wq[jn & 1], xq[jn & 1][tn], zero16, 0, 0, 0);
            /* the copies of the next iteration go out during the first five
             * slots, so they have the rest of the iteration to land */
            if (2 * k < NCOPY) copy_one(2 * k);
            if (2 * k + 1 < NCOPY) copy_one(2 * k + 1);
            if (j < valid) {
                const float dx = h2f(dxh[j & 1][ts]);
                const float dwf = dpp_source(h2f(dwh[j & 1]));
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ts][r] = fmac_row_lane(acc[ts][r], dwf, dx * (float)d[k & 1][r], r);
                if constexpr (DUMP) {
                    const int t = t0 + col + 32 * ts;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int n = n0 + 32 * wave + 8 * (r >> 2) + 4 * half + (r & 3);
                        if (t < a.M && n < work.N) a.dump[((size_t)t * work.N + n) * nblk + (size_t)(it * KB + j)] = d[k & 1][r];
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0070);                /* vmcnt(0): the next iteration has landed */
        __builtin_amdgcn_s_barrier();
    };
    for (int it = it0; it < niter; it += 2) {
        kstep(it, std::integral_constant<int, 0>{});
        if (it + 1 < niter) kstep(it + 1, std::integral_constant<int, 1>{});
    }

    /* lane: token t0 + col + 32 ts, rows n0 + 32 wave + 8 q + 4 half + (0..3) */
    const GemmOut o = work.out;
    const bool vec_ok = (o.ldc % 4 == 0) && (((uintptr_t)o.C) % 16 == 0) && (n0 + BN <= work.N);
#pragma unroll
    for (int ts = 0; ts < 2; ++ts) {
        const int t = t0 + col + 32 * ts;
        if (t >= a.M) continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n = n0 + 32 * wave + 8 * q + 4 * half;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = acc[ts][4 * q + i] + ((o.bias && n + i < work.N) ? o.bias[n + i] : 0.0f);
            float *dst = o.C + (size_t)t * o.ldc + n;
            if (vec_ok) *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            else {
#pragma unroll
                for (int i = 0; i < 4; ++i) if (n + i < work.N) dst[i] = v[i];
            }
        }
    }
}

int launch_gemm_q80_mfma(const void *A, const void *B, const float *bias, float *C,
                         int M, int N, int K, long ldc, const GemmOpts &opts, hipStream_t s)
{
    GemmArgs g = {};
    int32_t *const sums = opts.sums;
    g.dump = sums;
    g.ext_part = opts.scratch;
    g.ext_part_bytes = opts.scratch_bytes;
    g.A = (const uint8_t *)A; g.B = (const uint8_t *)B; g.bias = bias; g.C = C;
    g.M = M; g.N = N; g.nb = K / 32; g.ldc = ldc;
    /* lane offsets inside a tile are 32-bit */
    if ((long long)g.nb * 34 * GEMM8_BN >= (1ll << 31)) return (int)hipErrorInvalidValue;
    g.ntt = (M + GEMM8_BM - 1) / GEMM8_BM;
    g.nnt = (N + GEMM8_BN - 1) / GEMM8_BN;
    const int nnt8 = (g.nnt + 7) / 8 * 8;
#if CKQ_WITH_DUMP
    if (sums) return gemm_launch_split(gemm_q80_mfma_kernel<true>, g, (unsigned)(g.ntt * nnt8), (g.nb + GEMM8_KB - 1) / GEMM8_KB, s);
#else
    if (sums) return CKQ_ENODUMP;
#endif
    return gemm_launch_split(gemm_q80_mfma_kernel<false>, g, (unsigned)(g.ntt * nnt8), (g.nb + GEMM8_KB - 1) / GEMM8_KB, s);
}

int launch_gemm_q80_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s)
{
    if (gemm_group_tiles(in, M, GEMM8_BM) < GEMM_GROUP_MIN_TILES) return CKQ_ENOGROUP;
    GemmArgs g = {};
    g.A = (const uint8_t *)A; g.M = M; g.nb = K / 32;
    if ((long long)g.nb * 34 * GEMM8_BN >= (1ll << 31)) return (int)hipErrorInvalidValue;
    g.ntt = (M + GEMM8_BM - 1) / GEMM8_BM;
    return gemm_launch_grouped(gemm_q80_mfma_kernel<false>, g, in, s);
}
