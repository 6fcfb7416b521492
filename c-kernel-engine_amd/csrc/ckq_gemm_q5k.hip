/*
 * ckq_gemm_q5k.hip - prefill GEMM, Q5_K weights x Q8_K activations, on the
 * gfx950 int8 matrix cores.
 *
 *   C[t][n] = sum_b (dw(n,b) * dx(t,b)) * (float) I1 - (dmin(n,b) * dx(t,b)) * (float) I2   (+ bias[n])
 *   I1 = sum_{s<8} sc(n,b,s) * sum_{k in 32-run s} q5(n,k) * q8(t,k)                (exact int32)
 *   I2 = sum_{s<8} m(n,b,s) * (bsums(t,b,2s) + bsums(t,b,2s+1))                     (STORED bsums)
 * which is the reference's block routine (gemm_kernels_q5_k.c:130-208: two
 * integers per block, combined under the two fp32 scale products).
 *
 * Mapping to the hardware
 * - v_mfma_i32_32x32x32_i8: K = 32 is exactly one Q5_K sub-block.  The scaled
 *   weight v = sc * q5 <= 1953 is formed once per weight in 16-bit lanes
 *   (v_pk_mad_u16 on byte pairs, + 128) and split into two int8 planes
 *   v = 256 * H + L (L = signed low byte of v, H = high byte of v + 128), the
 *   byte lanes of the products gathered with v_perm_b32; both planes are
 *   accumulated over the block, I1 = 256 * IH + IL.
 * - The min term is two more int8 MFMAs per 32x32 tile per block: the eight
 *   bsum pairs of a token, split the same way into low and high bytes, fill 16
 *   of the 32 k slots of the token operand (the other 16 are zero); the weight
 *   operand holds the eight 6-bit mins in the low or in the high slots, giving
 *   sum m * PL and sum m * PH; I2 = 256 * that + this.
 * - Operands reach LDS by global->LDS loads only: a 176-byte block is eleven
 *   16-byte chunks; quants as in the Q4_K kernel (chunks XOR-swizzled by
 *   token); the tokens' block scales as 4-byte loads and their stored bsums as
 *   two 16-byte chunks each.  The loop holds no other memory operation, so a
 *   counted wait and a bare barrier end an iteration, and blocks are fetched two
 *   iterations ahead (three LDS stages, 121 KB).
 *
 * Block = 4 waves = 64 tokens x 128 weight rows; wave w owns rows 32w..32w+31.
 */
#include "ckq_gemm_common.hpp"
#include <atomic>
#include <type_traits>

constexpr int GEMM5_BM = 64, GEMM5_BN = 128, GEMM5_ROW = 176;

struct Gemm5Stage {
    uint8_t w[GEMM5_BN * GEMM5_ROW];   /* raw Q5_K blocks, row r at byte 176 r */
    uint8_t q[GEMM5_BM * 256];         /* int8 quants: 16-byte chunk c of token t in slot c ^ (t & 15) of its 256 bytes */
    uint8_t b[GEMM5_BM * 32];          /* stored bsums, 16 int16 per token */
    float   d[GEMM5_BM];               /* block scale of each token */
};

/* One 256-block of a tile.  The planes of slab s+1 are expanded between the
 * MFMAs of slab s; copy_one(i) issues one global->LDS copy of a later block. */
template <int NCOPY, bool DUMP, class CopyFn, class AfterFn>
__device__ __forceinline__ void gemm5_block(const uint8_t *w, const uint8_t *q, const uint8_t *bsum, const float *d, u32 wrow,
                                            const u32 (&aofs)[8], int col, int half, ckq_v16f (&acc)[2], CopyFn copy_one,
                                            AfterFn after_weights, const GemmDumpLane &dl)
{
#define CKQ_PIN() __builtin_amdgcn_sched_barrier(0)
    auto lds16 = [&](const void *p) { return *reinterpret_cast<const ckq_v4i *>(p); };
    const uint8_t *wr = w + wrow;

    /* raw block of this lane's row: header, fifth bits and nibbles its k-half touches */
    const ckq_v4i hv = lds16(wr);
    const ckq_v4i qh = lds16(wr + 16 + 16 * half);
    ckq_v4i qs[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) qs[g] = lds16(wr + 48 + 32 * g + 16 * half);

    ckq_v4i av[2][2];
    auto a_read = [&](int s) {
#pragma unroll
        for (int ts = 0; ts < 2; ++ts) av[s & 1][ts] = lds16(&q[aofs[s] + 32 * 256 * ts]);
    };
    a_read(0);

    /* token scales and stored bsums, read (through the integer vector type)
     * before the first copy is issued */
    float dx[2];      /* per token group: the block scale of the token of output (lane & 15) */
    ckq_v4i bs[2][2];
    const int dx_tok = mfma32_row_of_lane(col + 32 * half);
#pragma unroll
    for (int ts = 0; ts < 2; ++ts) {
        dx[ts] = __builtin_bit_cast(float, *reinterpret_cast<const int *>(&d[32 * ts + dx_tok]));
        bs[ts][0] = lds16(&bsum[(col + 32 * ts) * 32]);
        bs[ts][1] = lds16(&bsum[(col + 32 * ts) * 32 + 16]);
    }

    const u32 h0 = (u32)hv[0], h1 = (u32)hv[1], h2 = (u32)hv[2], h3 = (u32)hv[3];
    const u32 sc03 = h1 & 0x3f3f3f3fu;
    const u32 sc47 = (h3 & 0x0f0f0f0fu) | (((h1 >> 6) & 0x03030303u) << 4);
    const u32 mn03 = h2 & 0x3f3f3f3fu;
    const u32 mn47 = ((h3 >> 4) & 0x0f0f0f0fu) | (((h2 >> 6) & 0x03030303u) << 4);
    const float dw = h2f(h0 & 0xffff), dmin = h2f(h0 >> 16);

    u32 scp[2];
    ckq_v4i pL[2], pH[2];
    auto prep = [&](int s) {
        const u32 sc = ((s < 4 ? sc03 : sc47) >> (8 * (s & 3))) & 0xffu;
        scp[s & 1] = sc | (sc << 16);                                              /* sc in both 16-bit lanes */
    };
    auto decode = [&](int s, int i) {
        const int g = s >> 1, hi = s & 1;
        const u32 lw = (u32)qs[g][i], hw = (u32)qh[i];
        const u32 nib = hi ? ((lw >> 4) & 0x0f0f0f0fu) : (lw & 0x0f0f0f0fu);
        const u32 hb = (s == 0 ? hw : (hw >> s)) & 0x01010101u;                    /* fifth bit of element 32 s + l */
        const u32 q = (hb << 4) | nib;                                             /* four 5-bit values */
        const u32 e = __builtin_amdgcn_perm(0u, q, 0x0c020c00u);                   /* bytes 0, 2 in 16-bit lanes */
        const u32 o = __builtin_amdgcn_perm(0u, q, 0x0c030c01u);                   /* bytes 1, 3 */
        const u32 te = pk_mad_u16(e, scp[s & 1], 0x00800080u);                     /* sc * q + 128 */
        const u32 to = pk_mad_u16(o, scp[s & 1], 0x00800080u);
        pL[s & 1][i] = (int)(__builtin_amdgcn_perm(to, te, 0x06020400u) ^ 0x80808080u);
        pH[s & 1][i] = (int)__builtin_amdgcn_perm(to, te, 0x07030501u);
    };

    /* token operand of the min term: P_s = bsums[2s] + bsums[2s+1] (one dword
     * holds the pair), t = P + 128; bytes [PL_0..7 | PH_0..7] for the lanes of
     * k-half 0, zeros for k-half 1 */
    auto min_operand = [&](int ts) {
        u32 u[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const u32 d0 = (u32)bs[ts][p >> 1][2 * (p & 1)], d1 = (u32)bs[ts][p >> 1][2 * (p & 1) + 1];
            const u32 t0 = d0 + (d0 >> 16) + 128u, t1 = d1 + (d1 >> 16) + 128u;   /* low 16 bits: P + 128 */
            u[p] = __builtin_amdgcn_perm(t1, t0, 0x05040100u);                     /* [t0.lo16, t1.lo16] */
        }
        ckq_v4i a;
        a[0] = (int)(__builtin_amdgcn_perm(u[1], u[0], 0x06040200u) ^ 0x80808080u);   /* PL_0..3 */
        a[1] = (int)(__builtin_amdgcn_perm(u[3], u[2], 0x06040200u) ^ 0x80808080u);   /* PL_4..7 */
        a[2] = (int)__builtin_amdgcn_perm(u[1], u[0], 0x07050301u);                   /* PH_0..3 */
        a[3] = (int)__builtin_amdgcn_perm(u[3], u[2], 0x07050301u);                   /* PH_4..7 */
        if (half) a = ckq_v4i{0, 0, 0, 0};
        return a;
    };

    ckq_v16i iL[2], iH[2], mL[2], mH[2];
    const ckq_v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const ckq_v4i bM1 = {(int)mn03, (int)mn47, 0, 0}, bM2 = {0, 0, (int)mn03, (int)mn47};

    prep(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) decode(0, i);
    CKQ_PIN();
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        if (s < 7) prep(s + 1);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int ts = k >> 1;
            if ((k & 1) == 0) iL[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s & 1][ts], pL[s & 1], s == 0 ? zero16 : iL[ts], 0, 0, 0);
            else              iH[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s & 1][ts], pH[s & 1], s == 0 ? zero16 : iH[ts], 0, 0, 0);
            if (s == 0 && k == 0) {
                CKQ_PIN();
                after_weights();      /* the paired kernel: the weight image is in registers, it may take the next block */
                CKQ_PIN();
            }
            /* VALU work under this MFMA: a dword of the next slab's planes */
            if (s < 7) decode(s + 1, k);
            if (k == 0 && s < 7) a_read(s + 1);       /* operands of the next slab, three MFMAs ahead of their use */
            /* copies of a later block, spread over the slabs */
            if ((k & 1) == 0 && s + 4 * k < NCOPY) copy_one(s + 4 * k);
            CKQ_PIN();
        }
        /* the min term rides along in slabs 5 and 6, one token group each */
        if (s == 5 || s == 6) {
            const int ts = s - 5;
            const ckq_v4i aP = min_operand(ts);
            mL[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aP, bM1, zero16, 0, 0, 0);
            mH[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aP, bM2, zero16, 0, 0, 0);
            CKQ_PIN();
        }
    }

#pragma unroll
    for (int ts = 0; ts < 2; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i1 = (iH[ts][r] << 8) + iL[ts][r], i2 = (mH[ts][r] << 8) + mL[ts][r];
            const float f1 = (float)i1;
            const float f2 = (float)i2;
            acc[ts][r] = fmac_row_lane(acc[ts][r], dx[ts], dw * f1 - dmin * f2, r);
            if constexpr (DUMP) {
                const int tok = 32 * ts + 8 * (r >> 2) + (r & 3);
                dl.put(tok, 0, i1);
                dl.put(tok, 1, i2);
            }
        }
#undef CKQ_PIN
}

template <bool DUMP>
__global__ void __launch_bounds__(256, 1) gemm_q5k_mfma_kernel(GemmArgs a)
{
    constexpr int BM = GEMM5_BM, NST = 3;
    __shared__ __attribute__((aligned(16))) Gemm5Stage stage[NST];

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int col = lane & 31, half = lane >> 5;

    /* token tiles fastest inside an XCD, so each XCD's L2 sees a weight tile once */
    const GemmWork work = gemm_work(a, a.nb);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * GEMM5_BN;
    const u32 wstride = (u32)a.nb * 176u, xstride = (u32)a.nb * 292u;
    const int b0 = work.k0, b1 = work.k1, last = b1 - 1;
    const uint8_t *wbase = work.B + (size_t)n0 * wstride;       /* uniform */
    const uint8_t *xbase = a.A + (size_t)t0 * xstride;       /* uniform */

    /* Copy roles.  Weights: 128 rows x 11 chunks = 22 wave instructions, six
     * per wave (slots past 21 repeat slot 21: same bytes, no branch).  Quants:
     * four per wave.  Token scales: one 4-byte instruction, bsums: two 16-byte
     * chunks per token = two instructions; every wave issues one of each
     * (duplicates write the same bytes), which keeps the number of outstanding
     * copies equal in all waves. */
    constexpr int NWI = 6, NQI = 4, NCOPY = NWI + NQI + 2;
    u32 wofs_g[NWI], qofs_g[NQI], dofs_g, bofs_g;
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
        const int chunk = min(wave + 4 * i, 21) * 64 + lane, row = min(chunk / 11, work.N - 1 - n0), part = chunk % 11;
        wofs_g[i] = (u32)row * wstride + 16u * part;
    }
#pragma unroll
    for (int i = 0; i < NQI; ++i) {
        const int tl = 4 * (wave + 4 * i) + (lane >> 4), c = (lane & 15) ^ (tl & 15);
        qofs_g[i] = (u32)min(tl, a.M - 1 - t0) * xstride + 4u + 16u * c;
    }
    dofs_g = (u32)min(lane, a.M - 1 - t0) * xstride;
    {
        const int e = (wave & 1) * 64 + lane;                /* token e >> 1, chunk e & 1 of its bsums */
        bofs_g = (u32)min(e >> 1, a.M - 1 - t0) * xstride + 260u + 16u * (u32)(e & 1);
    }

    /* the copies address their source as buffer (uniform base in SGPRs) + per-lane
     * 32-bit offset + uniform K offset: no address arithmetic in the loop */
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_w = 0, cp_x = 0;
    int cp_buf = 0;
    auto copy_begin = [&](int b, int buf) {
        cp_w = b * 176;
        cp_x = b * 292;
        cp_buf = buf;
    };
    auto copy_one = [&](int i) {
        if (i < NWI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(stage[cp_buf].w + 1024 * min(wave + 4 * i, 21)), 16, (int)(wofs_g[i]), cp_w, 0, 0);
        else if (i < NWI + NQI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].q + 1024 * (wave + 4 * (i - NWI))), 16,
                                                     (int)qofs_g[i - NWI], cp_x, 0, 0);
        else if (i == NWI + NQI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].d), 4, (int)(dofs_g), cp_x, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].b + 1024 * (wave & 1)), 16, (int)(bofs_g), cp_x, 0, 0);
    };

    /* read-side offsets of this lane */
    const u32 wrow = (u32)(32 * wave + col) * (u32)GEMM5_ROW;
    u32 aofs[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) aofs[s] = (u32)col * 256u + 16u * (u32)((2 * s + half) ^ (col & 15));

    ckq_v16f acc[2];
#pragma unroll
    for (int ts = 0; ts < 2; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ts][r] = 0.0f;

#pragma unroll
    for (int p = 0; p < NST - 1; ++p) {
        copy_begin(min(b0 + p, last), p);
#pragma unroll
        for (int i = 0; i < NCOPY; ++i) copy_one(i);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);   /* vmcnt(0): this wave's copies have landed */
    __builtin_amdgcn_s_barrier();

    /* Block b+1 has landed when only the copies issued during this iteration
     * are still in flight; the block's waves exchange data only through those
     * copies, so a bare s_barrier follows. */
    /* One K-block; the stage it reads and the one it fills are compile-time
     * constants (the loop is unrolled over the stages), so LDS addresses are
     * per-lane registers set up once plus immediates. */
    auto kstep = [&](int b, auto curc) {
        constexpr int cur = decltype(curc)::value, pf = (cur + NST - 1) % NST;
        copy_begin(min(b + NST - 1, last), pf);
        __builtin_amdgcn_sched_barrier(0);
        GemmDumpLane dl = {};
        if constexpr (DUMP) {
            const int n = n0 + wave * 32 + col, tf = t0 + 4 * half;
            dl.tok_stride = gemm_opaque((size_t)work.N * a.nb * 2);
            dl.p = a.dump + ((size_t)tf * work.N + n) * a.nb * 2 + (size_t)b * 2;
            dl.tok_left = a.M - tf;
            dl.row_ok = n < work.N;
        }
        gemm5_block<NCOPY, DUMP>(stage[cur].w, stage[cur].q, stage[cur].b, stage[cur].d, wrow, aofs, col, half, acc, copy_one, [] {}, dl);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0070 | (NCOPY & 15) | ((NCOPY >> 4) << 14));
        __builtin_amdgcn_s_barrier();
    };
    static_assert(NST == 3, "the loop is unrolled over three stages");
    for (int b = b0; b < b1; b += 3) {
        kstep(b, std::integral_constant<int, 0>{});
        if (b + 1 < b1) kstep(b + 1, std::integral_constant<int, 1>{});
        if (b + 2 < b1) kstep(b + 2, std::integral_constant<int, 2>{});
    }

    const GemmOut o = work.out;
    const int n = n0 + wave * 32 + col;
    if (n < work.N) {
        const float bias = o.bias ? o.bias[n] : 0.0f;
#pragma unroll
        for (int ts = 0; ts < 2; ++ts)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * ts + 8 * (r >> 2) + 4 * half + (r & 3);
                if (t < a.M) gemm_store(&o.C[(size_t)t * o.ldc + n], acc[ts][r] + bias);
            }
    }
}

/* Two blocks per CU: ONE LDS image of the weights and two of the activations, bsums and scales (59 KB).  A lane takes
 * its row's whole raw block into registers at the start of a 256-block, so a barrier behind those reads frees the
 * image for the next block's weights; a second, independent block on the CU runs its MFMAs under this one's plane
 * expansion and fp32 combine and fills the waits of the shallower pipeline (a fetch has one iteration to land
 * instead of two).  Every LDS region is an object of its own: the compiler then puts no wait for a copy in front
 * of the reads of another region.  Same sums in the same order as gemm_q5k_mfma_kernel. */
template <bool DUMP>
__global__ void __launch_bounds__(256, 2) gemm_q5k_pair_kernel(GemmArgs a)
{
    constexpr int BM = GEMM5_BM;
    __shared__ __attribute__((aligned(16))) uint8_t wimg[GEMM5_BN * GEMM5_ROW];
    __shared__ __attribute__((aligned(16))) uint8_t q_even[BM * 256], q_odd[BM * 256];
    __shared__ __attribute__((aligned(16))) uint8_t b_even[BM * 32], b_odd[BM * 32];
    __shared__ __attribute__((aligned(16))) float d_even[BM], d_odd[BM];
    auto qst = [&](auto c) __attribute__((always_inline)) -> uint8_t * { if constexpr (decltype(c)::value == 0) return q_even; else return q_odd; };
    auto bst = [&](auto c) __attribute__((always_inline)) -> uint8_t * { if constexpr (decltype(c)::value == 0) return b_even; else return b_odd; };
    auto dst = [&](auto c) __attribute__((always_inline)) -> float * { if constexpr (decltype(c)::value == 0) return d_even; else return d_odd; };

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int col = lane & 31, half = lane >> 5;

    const GemmWork work = gemm_work(a, a.nb);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * GEMM5_BN;
    const u32 wstride = (u32)a.nb * 176u, xstride = (u32)a.nb * 292u;
    const int b0 = work.k0, b1 = work.k1, last = b1 - 1;
    const uint8_t *wbase = work.B + (size_t)n0 * wstride;
    const uint8_t *xbase = a.A + (size_t)t0 * xstride;

    /* copy roles as in gemm_q5k_mfma_kernel */
    constexpr int NWI = 6, NQI = 4, NCOPY = NWI + NQI + 2;
    u32 wofs_g[NWI], qofs_g[NQI], dofs_g, bofs_g;
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
        const int chunk = min(wave + 4 * i, 21) * 64 + lane, row = min(chunk / 11, work.N - 1 - n0), part = chunk % 11;
        wofs_g[i] = (u32)row * wstride + 16u * part;
    }
#pragma unroll
    for (int i = 0; i < NQI; ++i) {
        const int tl = 4 * (wave + 4 * i) + (lane >> 4), c = (lane & 15) ^ (tl & 15);
        qofs_g[i] = (u32)min(tl, a.M - 1 - t0) * xstride + 4u + 16u * c;
    }
    dofs_g = (u32)min(lane, a.M - 1 - t0) * xstride;
    {
        const int e = (wave & 1) * 64 + lane;
        bofs_g = (u32)min(e >> 1, a.M - 1 - t0) * xstride + 260u + 16u * (u32)(e & 1);
    }
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_w = 0, cp_x = 0;
    auto copy_begin = [&](int b) __attribute__((always_inline)) {
        cp_w = b * 176;
        cp_x = b * 292;
    };
    auto copy_one = [&](int i, auto bufc) __attribute__((always_inline)) {
        if (i < NWI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(wimg + 1024 * min(wave + 4 * i, 21)), 16, (int)(wofs_g[i]), cp_w, 0, 0);
        else if (i < NWI + NQI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(qst(bufc) + 1024 * (wave + 4 * (i - NWI))), 16,
                                                     (int)qofs_g[i - NWI], cp_x, 0, 0);
        else if (i == NWI + NQI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(dst(bufc)), 4, (int)(dofs_g), cp_x, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(bst(bufc) + 1024 * (wave & 1)), 16, (int)(bofs_g), cp_x, 0, 0);
    };

    const u32 wrow = (u32)(32 * wave + col) * (u32)GEMM5_ROW;
    u32 aofs[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) aofs[s] = (u32)col * 256u + 16u * (u32)((2 * s + half) ^ (col & 15));

    ckq_v16f acc[2];
#pragma unroll
    for (int ts = 0; ts < 2; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ts][r] = 0.0f;

    copy_begin(b0);
#pragma unroll
    for (int i = 0; i < NCOPY; ++i) copy_one(i, std::integral_constant<int, 0>{});
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();

    auto kstep = [&](int b, auto curc) __attribute__((always_inline)) {
        constexpr int cur = decltype(curc)::value;
        GemmDumpLane dl = {};
        if constexpr (DUMP) {
            const int n = n0 + wave * 32 + col, tf = t0 + 4 * half;
            dl.tok_stride = gemm_opaque((size_t)work.N * a.nb * 2);
            dl.p = a.dump + ((size_t)tf * work.N + n) * a.nb * 2 + (size_t)b * 2;
            dl.tok_left = a.M - tf;
            dl.row_ok = n < work.N;
        }
        auto after_weights = [&]() __attribute__((always_inline)) {
            __builtin_amdgcn_s_waitcnt(0xc07f);      /* lgkmcnt(0): this wave's reads of the images have returned */
            __builtin_amdgcn_s_barrier();
            copy_begin(min(b + 1, last));
        };
        auto copy_next = [&](int i) __attribute__((always_inline)) { copy_one(i, std::integral_constant<int, cur ^ 1>{}); };
        __builtin_amdgcn_sched_barrier(0);
        gemm5_block<NCOPY, DUMP>(wimg, qst(curc), bst(curc), dst(curc), wrow, aofs, col, half, acc, copy_next, after_weights, dl);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
    };
    for (int b = b0; b < b1; b += 2) {
        kstep(b, std::integral_constant<int, 0>{});
        if (b + 1 < b1) kstep(b + 1, std::integral_constant<int, 1>{});
    }

    const GemmOut o = work.out;
    const int n = n0 + wave * 32 + col;
    if (n < work.N) {
        const float bias = o.bias ? o.bias[n] : 0.0f;
#pragma unroll
        for (int ts = 0; ts < 2; ++ts)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * ts + 8 * (r >> 2) + 4 * half + (r & 3);
                if (t < a.M) gemm_store(&o.C[(size_t)t * o.ldc + n], acc[ts][r] + bias);
            }
    }
}

/* More tiles than CUs: the paired kernel (512 x 11008, K = 4096: 99.2 -> 85.3 us; 2048 tokens: 374 -> 320; 512 x 8192:
 * 67.9 -> 60.4); up to one tile per CU the three-stage kernel, whose deeper pipeline serves a block that has its CU to
 * itself (256 tiles: 81.7 against 83.0).  variant: 0 = by tile count, 1 = one block per CU always, 2 = paired always. */
static std::atomic<int> g_q5k_variant{0};
extern "C" void ckq_launch_set_q5k_variant(int variant) { g_q5k_variant.store(variant == 1 || variant == 2 ? variant : 0); }
static bool q5k_take_pair(int tiles)
{
    const int forced = g_q5k_variant.load(std::memory_order_relaxed);
    return forced ? forced == 2 : tiles > 256;
}

int launch_gemm_q5k_mfma(const void *A, const void *B, const float *bias, float *C,
                         int M, int N, int K, long ldc, const GemmOpts &opts, hipStream_t s)
{
    GemmArgs g = {};
    int32_t *const sums = opts.sums;
    g.dump = sums;
    g.ext_part = opts.scratch;
    g.ext_part_bytes = opts.scratch_bytes;
    g.A = (const uint8_t *)A; g.B = (const uint8_t *)B; g.bias = bias; g.C = C;
    g.M = M; g.N = N; g.nb = K / 256; g.ldc = ldc;
    /* lane offsets inside a tile are 32-bit */
    if ((long long)g.nb * 292 * 128 >= (1ll << 31)) return (int)hipErrorInvalidValue;
    g.ntt = (M + GEMM5_BM - 1) / GEMM5_BM;
    g.nnt = (N + GEMM5_BN - 1) / GEMM5_BN;
    const int nnt8 = (g.nnt + 7) / 8 * 8;
    if (q5k_take_pair(g.ntt * g.nnt)) {
#if CKQ_WITH_DUMP
        if (sums) return gemm_launch_split(gemm_q5k_pair_kernel<true>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
#else
        if (sums) return CKQ_ENODUMP;
#endif
        return gemm_launch_split(gemm_q5k_pair_kernel<false>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
    }
#if CKQ_WITH_DUMP
    if (sums) return gemm_launch_split(gemm_q5k_mfma_kernel<true>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
#else
    if (sums) return CKQ_ENODUMP;
#endif
    return gemm_launch_split(gemm_q5k_mfma_kernel<false>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
}

int launch_gemm_q5k_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s)
{
    if (gemm_group_tiles(in, M, GEMM5_BM) < GEMM_GROUP_MIN_TILES) return CKQ_ENOGROUP;
    GemmArgs g = {};
    g.A = (const uint8_t *)A; g.M = M; g.nb = K / 256;
    if ((long long)g.nb * 292 * 128 >= (1ll << 31)) return (int)hipErrorInvalidValue;
    g.ntt = (M + GEMM5_BM - 1) / GEMM5_BM;
    if (q5k_take_pair(gemm_group_tiles(in, M, GEMM5_BM))) return gemm_launch_grouped(gemm_q5k_pair_kernel<false>, g, in, s);
    return gemm_launch_grouped(gemm_q5k_mfma_kernel<false>, g, in, s);
}
