/*
 * ckq_gemm_q4k_t96.hip - prefill GEMM, Q4_K weights x Q8_K activations, on tiles of 128 weight rows x 96
 * tokens: the arithmetic and the operand paths of ckq_gemm_q4k.hip (two int8 planes per weight, the min
 * term as one bf16 MFMA per 32x32 tile and block, everything through LDS by global->LDS loads), with
 * three 32-token groups per wave instead of two.  The two planes of a wave's 32 rows are expanded once
 * per 256-block and serve 48 int8 MFMAs instead of 32, so the loop issues about 8.5 VALU instructions per
 * MFMA instead of 9.8 (whole launches, by the counters: 10.3 instead of 11.7), and the weights are read
 * from LDS once per 96 tokens instead of once per 64.
 *
 * What pays for it: the planes of all eight sub-blocks stay in registers across the three groups (64
 * registers), two sets of int32 accumulators are alive at once (a group's fp32 combine runs under the
 * next group's MFMAs, the last group's under the first MFMAs of the next 256-block), and LDS holds ONE
 * image of the weights - a wave reads its rows' raw blocks at the start of a 256-block, a barrier follows,
 * and the next block's weights are copied in behind it - beside two images of the activations and the
 * tokens' scales and bsums as stored: 74.6 KB, two blocks per CU.
 *
 * A token tile that is not full computes only the groups that hold tokens (1, 2 or 3; uniform per
 * block), and such tiles get the last block ids of their XCD, so that what starts late is short.
 */
#include "ckq_gemm_q4k.hpp"
#include <type_traits>

constexpr int T96_BM = 96;
constexpr int T96_BN = GEMM_TILE_ROWS;

/* Token scales and bsums of one 256-block of 96 tokens: as stored (filled by global->LDS copies; the second
 * 4-byte copy of the scales covers 64 lanes, hence 128 slots) and as the kernel reads them. */
struct T96Raw {
    uint8_t bs[T96_BM * 32];     /* sixteen int16 per token */
    float   d[128];
};
struct T96Side {
    float    d[T96_BM];          /* block scale of each token */
    uint16_t b[T96_BM * 16];     /* bf16: lo_0..7, 64*hi_0..7 of the pair sums of the stored bsums */
};

/* The last token group of a 256-block, MFMAs done but not yet combined into the fp32 accumulators: that happens
 * under the MFMAs of the next block's first group (or after the loop).  All zero before the first block. */
struct T96Carry {
    ckq_v16i H, L;       /* int32 sums of the two planes */
    ckq_v16f i2;         /* min term */
    float dw, dmin, dx;  /* the row's two block scales; the token scale of this lane's output (lane & 15) */
};

/* acc[r] += dx(token of r) * (dw * (8 H[r] + L[r]) - dmin * i2[r]); tok0 = first token of the group (dump builds) */
template <bool DUMP>
__device__ __forceinline__ void t96_combine(ckq_v16f &acc, const ckq_v16i &H, const ckq_v16i &L, const ckq_v16f &i2, float dw, float dmin,
                                            float dx, int r, const GemmDumpLane &dl, int tok0)
{
    const int i1 = (H[r] << 3) + L[r];
    const float f = (float)i1;
    const float u = dw * f - dmin * i2[r];
    acc[r] = fmac_row_lane(acc[r], dx, u, r);
    if constexpr (DUMP) {
        const int tok = tok0 + 8 * (r >> 2) + (r & 3);
        dl.put(tok, 0, i1);
        dl.put(tok, 1, (int)i2[r]);
    }
}

/* One 256-block of NG 32-token groups.  Steps s = 0 .. 8 NG - 1: group s / 8, sub-block s % 8, two MFMAs
 * each (plane H, plane L).  Under group 0 the planes of sub-blocks 1..7 are expanded, one per step, and the
 * last group of the PREVIOUS block (`carry`) is combined - its first four outputs while the reads of the weight
 * image are in flight; under group g > 0 the outputs of group g - 1 are combined, two per step.  The last
 * group of this block leaves in `carry`.  side_begin() starts the reads of the raw side data; after_weights()
 * runs once the first MFMA is issued: it stores the side data in the MFMA's form, waits for this wave's reads
 * of the weight image and joins the block's barrier; copy_one(i) issues the i-th global->LDS copy of the next
 * block.  dlp: where a dump build stores the sums of the previous block. */
template <int NG, bool DUMP, class CopyFn, class BeginFn, class AfterFn>
__device__ __forceinline__ void t96_block_pipe(const uint8_t *w, const uint8_t *q, const T96Side &sd, u32 wofs, const u32 (&aofs)[8], int col, int half,
                                               ckq_v16f (&acc)[3], T96Carry &carry, CopyFn copy_one, BeginFn side_begin, AfterFn after_weights,
                                               const GemmDumpLane &dl, const GemmDumpLane &dlp)
{
#define CKQ_PIN() __builtin_amdgcn_sched_barrier(0)
    constexpr int NS = 8 * NG;
    constexpr int NCOPY = 5 + 2 * NG + 1, COPIES_PER_STEP = (NCOPY + NS - 2) / (NS - 1);
    auto lds16 = [&](const uint8_t *p) { return *reinterpret_cast<const ckq_v4i *>(p); };
    auto a_read = [&](int s) { return lds16(&q[aofs[s & 7] + 32 * 256 * (s >> 3)]); };
    auto combine_prev = [&](int r) { t96_combine<DUMP>(acc[NG - 1], carry.H, carry.L, carry.i2, carry.dw, carry.dmin, carry.dx, r, dlp, 32 * (NG - 1)); };

    const ckq_v4i hv = lds16(&w[wofs]);
    ckq_v4i qv[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) qv[g] = lds16(&w[wofs + 16 + 32 * g + 16 * half]);
    ckq_v4i av[2];
    av[0] = a_read(0);
    side_begin();
    CKQ_PIN();
#pragma unroll
    for (int r = 0; r < 4; ++r) combine_prev(r);
    CKQ_PIN();

    const u32 h0 = (u32)hv[0], h1 = (u32)hv[1], h2 = (u32)hv[2], h3 = (u32)hv[3];
    const u32 sc03 = h1 & 0x3f3f3f3fu;
    const u32 sc47 = (h3 & 0x0f0f0f0fu) | (((h1 >> 6) & 0x03030303u) << 4);
    float dw = h2f(h0 & 0xffff);
    const float dmin = h2f(h0 >> 16);
    asm volatile("" : "+v"(dw));      /* a float of its own: see gemm_block_pipe */

    const u32 schi03 = (sc03 >> 3) & 0x07070707u, sclo03 = sc03 & 0x07070707u;
    const u32 schi47 = (sc47 >> 3) & 0x07070707u, sclo47 = sc47 & 0x07070707u;
    auto pair_of_byte = [](u32 v, int k) { return __builtin_amdgcn_perm(0u, v, 0x0c000c00u | (u32)k | ((u32)k << 16)); };

    ckq_v4i bH[8], bL[8];
    auto decode = [&](int j) {
        const int g = j >> 1, hi = j & 1;
        const u32 mh = pair_of_byte(j < 4 ? schi03 : schi47, j & 3), ml = pair_of_byte(j < 4 ? sclo03 : sclo47, j & 3);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 v = (u32)qv[g][i];
            const u32 nib = hi ? ((v >> 4) & 0x0f0f0f0fu) : (v & 0x0f0f0f0fu);
            bH[j][i] = mul_bytes(nib, mh);
            bL[j][i] = mul_bytes(nib, ml);
        }
    };
    decode(0);

    ckq_v16i cH[NG], cL[NG];
    const ckq_v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    ckq_v8bf bm;
    ckq_v4i ab;
    float dxl[NG];
    ckq_v16f i2;
    auto combine = [&](int g, int r) { t96_combine<DUMP>(acc[g], cH[g], cL[g], i2, dw, dmin, dxl[g], r, dl, 32 * g); };
    const int dx_tok = mfma32_row_of_lane(col + 32 * half);

    CKQ_PIN();
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int g = s >> 3, j = s & 7;
        if (s + 1 < NS) av[(s + 1) & 1] = a_read(s + 1);
        cH[g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s & 1], bH[j], j == 0 ? zero16 : cH[g], 0, 0, 0);
        CKQ_PIN();
        if (s == 0) {
            after_weights();
            CKQ_PIN();
        }
        if (g == 0) {
            if (j < 7) decode(j + 1);
            else {
                /* the eight mins as bf16 */
                const u32 mn03 = h2 & 0x3f3f3f3fu;
                const u32 mn47 = ((h3 >> 4) & 0x0f0f0f0fu) | (((h2 >> 6) & 0x03030303u) << 4);
                u32 m[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32 src = i < 2 ? mn03 : mn47;
                    const u32 m0 = (src >> (16 * (i & 1))) & 0xff, m1 = (src >> (16 * (i & 1) + 8)) & 0xff;
                    m[i] = bf16_pair((float)m0, (float)m1);
                }
                const ckq_v4i t = {(int)m[0], (int)m[1], (int)m[2], (int)m[3]};
                bm = __builtin_bit_cast(ckq_v8bf, t);
            }
            if (4 + 2 * j < 16) combine_prev(4 + 2 * j);
        } else combine(g - 1, 2 * j);
        CKQ_PIN();
        cL[g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s & 1], bL[j], j == 0 ? zero16 : cL[g], 0, 0, 0);
        if (s >= 1) {
#pragma unroll
            for (int c = 0; c < COPIES_PER_STEP; ++c)
                if ((s - 1) * COPIES_PER_STEP + c < NCOPY) copy_one((s - 1) * COPIES_PER_STEP + c);
        }
        if (g == 0) {
            if (5 + 2 * j < 16) combine_prev(5 + 2 * j);
        } else combine(g - 1, 2 * j + 1);
        if (j == 5) ab = lds16(reinterpret_cast<const uint8_t *>(&sd.b[(32 * g + col) * 16 + 8 * half]));
        if (j == 6) dxl[g] = __builtin_bit_cast(float, *reinterpret_cast<const int *>(&sd.d[32 * g + dx_tok]));
        if (j == 7) {
            ckq_v16f zero;
#pragma unroll
            for (int r = 0; r < 16; ++r) zero[r] = 0.0f;
            i2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(ckq_v8bf, ab), bm, zero, 0, 0, 0);
        }
        CKQ_PIN();
    }
    carry.H = cH[NG - 1];
    carry.L = cL[NG - 1];
    carry.i2 = i2;
    carry.dw = dw;
    carry.dmin = dmin;
    carry.dx = dxl[NG - 1];
#undef CKQ_PIN
}

template <int WPE, bool DUMP = false>
__global__ void __launch_bounds__(256, DUMP ? 1 : WPE) gemm_q4k_t96_kernel(GemmArgs a)
{
    constexpr int BM = T96_BM;
    /* every LDS region is an object of its own: a copy into one cannot meet a read of another, and the
     * compiler puts no wait for the copy in front of such a read */
    __shared__ __attribute__((aligned(16))) uint8_t wst[T96_BN * 144];     /* raw Q4_K blocks, row r at byte 144 r */
    __shared__ __attribute__((aligned(16))) uint8_t q_even[BM * 256], q_odd[BM * 256];
    __shared__ __attribute__((aligned(16))) T96Raw raw;                    /* next block's token scales and bsums as stored */
    __shared__ __attribute__((aligned(16))) T96Side side;                  /* this block's, as the MFMA wants them */
    auto qst = [&](auto bufc) __attribute__((always_inline)) -> uint8_t * {
        if constexpr (decltype(bufc)::value == 0) return q_even; else return q_odd;
    };

    const int wave = wave_in_block();
    const int tid = threadIdx.x, lane = tid & 63;
    const int col = lane & 31, half = lane >> 5;

    /* tile of this block: full token tiles first (token tiles fastest, so neighbours share weights), then
     * the partial token tile of every weight-row tile */
    const GemmWork work = gemm_work(a, a.nb);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int nfull = a.M / BM, ncg = (work.nnt + 7) >> 3;
    int cg, tt;
    if (seq < ncg * nfull) { cg = seq / nfull; tt = seq - cg * nfull; }
    else { cg = seq - ncg * nfull; tt = nfull; }
    const int nt = cg * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * T96_BN;
    const int ng = min(3, (a.M - t0 + 31) >> 5);
    const int tlim = a.M - 1 - t0;                 /* last token of the matrix, counted from t0 */
    const u32 wstride = (u32)a.nb * 144u, xstride = (u32)a.nb * 292u;
    const int b0 = work.k0, b1 = work.k1, last = b1 - 1;
    const uint8_t *wbase = work.B + (size_t)n0 * wstride;
    const uint8_t *xbase = a.A + (size_t)t0 * xstride;

    /* copy roles: weights and quants as in gemm_q4k_mfma_kernel (six instead of four quant copies per wave);
     * the 36 bytes of scale and bsums of every token come as they are stored - waves 0-2 one 16-byte
     * copy each (two chunks per token), wave 3 two 4-byte copies (the scales) */
    constexpr int NWI = 5, NQI = BM / 16;
    u32 wofs_g[NWI], qofs_g[NQI], sofs, sofs2;
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
        const int chunk = min(wave + 4 * i, 17) * 64 + lane, row = min(chunk / 9, work.N - 1 - n0), part = chunk % 9;
        wofs_g[i] = (u32)row * wstride + 16u * part;
    }
#pragma unroll
    for (int i = 0; i < NQI; ++i) {
        const int tl = 4 * (wave + 4 * i) + (lane >> 4), c = (lane & 15) ^ (tl & 15);
        qofs_g[i] = (u32)min(tl, tlim) * xstride + 4u + 16u * c;
    }
    {
        const int c = 64 * min(wave, 2) + lane;
        sofs  = wave < 3 ? (u32)min(c >> 1, tlim) * xstride + 260u + 16u * (c & 1) : (u32)min(lane, tlim) * xstride;
        sofs2 = (u32)min(64 + (lane & 31), tlim) * xstride;
    }
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_w = 0, cp_x = 0;
    auto copy_begin = [&](int b) __attribute__((always_inline)) {
        cp_w = b * 144;
        cp_x = b * 292;
    };
    /* copy i of a block: 0..4 weights, 5..5+2NG-1 quants (the stage is a compile-time constant), then the raw side data */
    auto copy_one = [&](int i, int nq, auto bufc) __attribute__((always_inline)) {
        if (i < NWI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(wst + 1024 * min(wave + 4 * i, 17)), 16,
                                                     (int)wofs_g[i], cp_w, 0, 0);
        else if (i < NWI + nq)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(qst(bufc) + 1024 * (wave + 4 * (i - NWI))), 16,
                                                     (int)qofs_g[i - NWI], cp_x, 0, 0);
        else if (wave < 3)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(raw.bs + 1024 * wave), 16, (int)sofs, cp_x, 0, 0);
        else {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(raw.d), 4, (int)sofs, cp_x, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(raw.d + 64), 4, (int)sofs2, cp_x, 0, 0);
        }
    };
    /* raw -> side, four threads per token (tokens 64..95: the first 128 threads once more): the scale as it is, the
     * sixteen bsums as eight pair sums split lo + 64 hi, both exact in bf16 */
    const int st_tok = tid >> 2, st_q = tid & 3;
    const bool st_two = wave < 2 && ng == 3;
    auto side_read = [&](int tok, u32 (&bs)[2], u32 &d) __attribute__((always_inline)) {
        const u32 *p = reinterpret_cast<const u32 *>(raw.bs + tok * 32 + 8 * st_q);
        bs[0] = p[0];
        bs[1] = p[1];
        d = reinterpret_cast<const u32 *>(raw.d)[tok];
    };
    auto side_put = [&](int tok, const u32 (&bs)[2], u32 d) __attribute__((always_inline)) {
        if (st_q == 0) reinterpret_cast<u32 *>(side.d)[tok] = d;
        const int s0 = (int)(int16_t)(bs[0] & 0xffff) + (int)(int16_t)(bs[0] >> 16);
        const int s1 = (int)(int16_t)(bs[1] & 0xffff) + (int)(int16_t)(bs[1] >> 16);
        u32 *bd = reinterpret_cast<u32 *>(&side.b[tok * 16]);
        bd[st_q]     = bf16_pair((float)(s0 & 63), (float)(s1 & 63));
        bd[4 + st_q] = bf16_pair((float)(64 * (s0 >> 6)), (float)(64 * (s1 >> 6)));
    };

    const u32 wofs_l = (u32)(32 * wave + col) * 144u;
    u32 aofs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) aofs[j] = (u32)col * 256u + 16u * (u32)((2 * j + half) ^ (col & 15));

    ckq_v16f acc[3];
#pragma unroll
    for (int g = 0; g < 3; ++g)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[g][r] = 0.0f;

    auto run = [&](auto ngc) __attribute__((always_inline)) {
        constexpr int NG = decltype(ngc)::value;
        constexpr int NCOPY = NWI + 2 * NG + 1;
        T96Carry carry;
#pragma unroll
        for (int r = 0; r < 16; ++r) { carry.H[r] = 0; carry.L[r] = 0; carry.i2[r] = 0.0f; }
        carry.dw = carry.dmin = carry.dx = 0.0f;
        auto dump_lane = [&](int b, bool ok) __attribute__((always_inline)) {
            GemmDumpLane dl = {};
            if constexpr (DUMP) {
                const int n = n0 + wave * 32 + col, tf = t0 + 4 * half;
                dl.tok_stride = gemm_opaque((size_t)work.N * a.nb * 2);
                dl.p = a.dump + ((size_t)tf * work.N + n) * a.nb * 2 + (ptrdiff_t)b * 2;
                dl.tok_left = a.M - tf;
                dl.row_ok = n < work.N && ok;
            }
            return dl;
        };
        copy_begin(b0);
#pragma unroll
        for (int i = 0; i < NCOPY; ++i) copy_one(i, 2 * NG, std::integral_constant<int, 0>{});
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();

        auto kstep = [&](int b, auto curc) __attribute__((always_inline)) {
            constexpr int cur = decltype(curc)::value;
            const GemmDumpLane dl = dump_lane(b, true), dlp = dump_lane(b - 1, b > b0);
            /* start of a block: this thread's share of the side data, raw */
            u32 bs[2], bs2[2] = {0, 0}, sd, sd2 = 0;
            auto side_begin = [&]() __attribute__((always_inline)) {
                side_read(st_tok, bs, sd);
                if (st_two) side_read(64 + st_tok, bs2, sd2);
            };
            /* once the first MFMA is out: the side data in the MFMA's form, then the barrier behind which every wave
             * has its rows of the weight image in registers and the side data of the block is complete; the weight
             * image and the raw side data then take the next block */
            auto after_weights = [&]() __attribute__((always_inline)) {
                side_put(st_tok, bs, sd);
                if (st_two) side_put(64 + st_tok, bs2, sd2);
                __builtin_amdgcn_s_waitcnt(0xc07f);      /* lgkmcnt(0): the reads have returned */
                __syncthreads();
                copy_begin(min(b + 1, last));
            };
            auto copy_next = [&](int i) __attribute__((always_inline)) { copy_one(i, 2 * NG, std::integral_constant<int, cur ^ 1>{}); };
            __builtin_amdgcn_sched_barrier(0);
            t96_block_pipe<NG, DUMP>(wst, qst(curc), side, wofs_l, aofs, col, half, acc, carry, copy_next, side_begin, after_weights, dl, dlp);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0x0070);
            __syncthreads();
        };
        for (int b = b0; b < b1; b += 2) {
            kstep(b, std::integral_constant<int, 0>{});
            if (b + 1 < b1) kstep(b + 1, std::integral_constant<int, 1>{});
        }
        /* the last group of the last block */
        const GemmDumpLane dll = dump_lane(last, true);
#pragma unroll
        for (int r = 0; r < 16; ++r)
            t96_combine<DUMP>(acc[NG - 1], carry.H, carry.L, carry.i2, carry.dw, carry.dmin, carry.dx, r, dll, 32 * (NG - 1));
    };
    if (ng == 3) run(std::integral_constant<int, 3>{});
    else if (ng == 2) run(std::integral_constant<int, 2>{});
    else run(std::integral_constant<int, 1>{});

    const GemmOut o = work.out;
    const int n = n0 + wave * 32 + col;
    if (n < work.N) {
        const float bias = o.bias ? o.bias[n] : 0.0f;
#pragma unroll
        for (int g = 0; g < 3; ++g)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * g + 8 * (r >> 2) + 4 * half + (r & 3);
                if (t < a.M) gemm_store(&o.C[(size_t)t * o.ldc + n], acc[g][r] + bias);
            }
    }
}

int gemm_q4k_t96_token_tiles(int M) { return (M + T96_BM - 1) / T96_BM; }

/* g: A, B, bias, C, M, N, nb, ldc, nnt and the dump pointer set; the token tiling is set here.
 * One block per tile, no K split: for launches whose tiles fill the chip. */
int launch_gemm_q4k_t96(GemmArgs g, hipStream_t s)
{
    g.ntt = gemm_q4k_t96_token_tiles(g.M);
    g.ngroup = 0; g.splits = 1; g.k_per = 0; g.part = nullptr;
    const unsigned grid = (unsigned)g.ntt * (unsigned)((g.nnt + 7) / 8 * 8);
    if (g.dump) {
#if CKQ_WITH_DUMP
        hipLaunchKernelGGL((gemm_q4k_t96_kernel<CKQ_GEMM_WPE, true>), dim3(grid), dim3(256), 0, s, g);
        return (int)hipGetLastError();
#else
        return CKQ_ENODUMP;
#endif
    }
    hipLaunchKernelGGL((gemm_q4k_t96_kernel<CKQ_GEMM_WPE, false>), dim3(grid), dim3(256), 0, s, g);
    return (int)hipGetLastError();
}

/* The matrices of `in` against the same activations as one grid of 96-token tiles; g: A, M, nb set. */
int launch_gemm_q4k_t96_group(GemmArgs g, const GemmGroupIn &in, hipStream_t s)
{
    g.ntt = gemm_q4k_t96_token_tiles(g.M);
    return gemm_launch_grouped(gemm_q4k_t96_kernel<CKQ_GEMM_WPE, false>, g, in, s, 256);
}
