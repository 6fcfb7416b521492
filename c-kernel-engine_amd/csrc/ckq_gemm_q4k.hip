/*
 * ckq_gemm_q4k.hip - prefill GEMM, Q4_K weights x Q8_K activations, on the
 * gfx950 int8 matrix cores.
 *
 *   C[t][n] = sum_b dx(t,b) * ( dw(n,b) * I1(t,n,b) - dmin(n,b) * I2(t,n,b) ) (+ bias[n])
 *   I1 = sum_j sc(n,b,j) * sum_{k in sub-block j} q4(n,k) * q8(t,k)      (exact int32)
 *   I2 = sum_j m(n,b,j)  * (bsums(t,b,2j) + bsums(t,b,2j+1))             (STORED bsums)
 * which is the arithmetic of the reference's token loop over
 * gemv_q4_k_q8_k (gemm_kernels_q4k_q8k.c:121-181, 283-326) with the integer
 * parts kept exact and one fp32 rounding sequence per 256-element block.
 *
 * Mapping to the hardware
 * - v_mfma_i32_32x32x32_i8: K = 32 is exactly one Q4_K sub-block.  A = 32
 *   tokens x 32 k (int8 activations), B = 32 k x 32 weight rows, D = 32x32
 *   int32.  Lane l supplies row/column l%32 and the 16 k of half l/32.
 * - The 6-bit sub-block scale cannot ride in an int8 operand (sc*q4 <= 945),
 *   and applying it to the int32 outputs costs one VALU op per output per
 *   sub-block, more than the MFMA itself.  Instead the weights are expanded to
 *   TWO int8 planes, H = (sc>>3)*q4 and L = (sc&7)*q4 (both <= 105), each
 *   accumulated over all eight sub-blocks of a block; I1 = 8*H + L exactly.
 *   Nibble unpack and the two multiplies (v_pk_mul_lo_u16 on byte pairs) are
 *   done once per weight and reused for both 32-token halves of the tile.
 * - The min term contracts 8 (min, bsum) pairs per block.  Stored bsums need
 *   13 bits; split as lo + 64*hi (lo in [0,63], hi in [-64,63]) both parts and
 *   the 6-bit mins are exact in bf16, so ONE v_mfma_f32_32x32x16_bf16 per
 *   32x32 tile per block yields I2 exactly in fp32 (|I2| < 2^24).
 * - Every operand reaches the matrix cores through LDS, filled by 16-byte
 *   global->LDS loads (no VGPR staging): the raw Q4_K blocks of the tile's
 *   128 rows (9 consecutive lanes read one 144-byte block contiguously) and
 *   the int8 quants of its 64 tokens (16 lanes per token), double-buffered
 *   against the MFMA work.  A lane reads its own row's header and nibble
 *   runs back with ds_read_b128 (144-byte stride: conflict-free); the quants
 *   are stored with their 16-byte chunks XOR-swizzled by the token number so
 *   that 32 token rows at a 256-byte stride read conflict-free too.
 *
 * Block = 4 waves = 64 tokens x 128 weight rows; wave w owns rows
 * 32w..32w+31.  Grid: token tiles fastest inside an XCD so the eight XCD L2s
 * each see a weight tile once.
 */
#include "ckq_gemm_q4k.hpp"
#include <atomic>
#include <type_traits>

constexpr int GEMM_BM = 64;     /* tokens per tile */
constexpr int GEMM_BN = GEMM_TILE_ROWS;    /* weight rows per tile */

/* LDS image of one 256-block for a tile of 128 weight rows x 64 tokens. */
struct GemmStage {
    uint8_t  w[GEMM_BN * 144];    /* raw Q4_K blocks, row r at byte 144 r */
    uint8_t  q[GEMM_BM * 256];    /* int8 quants: 16-byte chunk c of token t in slot c ^ (t & 15) of its 256 bytes */
    float    d[GEMM_BM];          /* block scale of each token */
    uint16_t b[GEMM_BM * 16];     /* bf16: lo_0..7, 64*hi_0..7 of the stored bsums */
};

/* One 256-block of a 64-token tile, software-pipelined by hand.  The 32 int8
 * MFMAs run in four passes of eight - (tokens 0-31 | 32-63) x (sub-blocks 0-3 |
 * 4-7) - so that VALU work always has matrix work to hide under: the planes
 * of sub-blocks 0-3 are expanded during pass 1, those of 4-7 during pass 2,
 * and the fp32 combine of tokens 0-31 runs under pass 4.  Activation operands
 * are read from LDS two steps ahead.  Scheduling barriers pin that order. */
template <bool DUMP, class CopyFn>
__device__ __forceinline__ void gemm_block_pipe(const GemmStage &st, u32 wofs, const u32 (&aofs)[8], int col, int half,
                                                ckq_v16f (&acc)[2], CopyFn copy_one, const GemmDumpLane &dl)
{
#define CKQ_PIN() __builtin_amdgcn_sched_barrier(0)
    auto lds16 = [&](const uint8_t *p) { return *reinterpret_cast<const ckq_v4i *>(p); };
    /* step s = 0..15: pass order (ts, j) = (0,0..3) (1,0..3) (0,4..7) (1,4..7) */
    auto step_ts = [](int s) { return (s >> 2) & 1; };
    auto step_j  = [](int s) { return (s & 3) | ((s >> 3) << 2); };
    auto a_read = [&](int s) { return lds16(&st.q[aofs[step_j(s)] + 32 * 256 * step_ts(s)]); };

    const ckq_v4i hv = lds16(&st.w[wofs]);
    ckq_v4i qv[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) qv[g] = lds16(&st.w[wofs + 16 + 32 * g + 16 * half]);
    ckq_v4i av[3];
    av[0] = a_read(0);
    av[1] = a_read(1);

    const u32 h0 = (u32)hv[0], h1 = (u32)hv[1], h2 = (u32)hv[2], h3 = (u32)hv[3];
    const u32 sc03 = h1 & 0x3f3f3f3fu;
    const u32 sc47 = (h3 & 0x0f0f0f0fu) | (((h1 >> 6) & 0x03030303u) << 4);
    float dw = h2f(h0 & 0xffff);
    const float dmin = h2f(h0 >> 16);
    /* dw as a float of its own: folded into the combine as an fp16 operand (v_fma_mix) its result would need
     * a wait state in front of every lane-broadcast multiply-add that consumes it */
    asm volatile("" : "+v"(dw));

    /* the two 3-bit halves of the eight scales, four per word; byte k of a word
     * becomes the u16 pair {k-th, k-th} a plane is multiplied by with one v_perm_b32
     * (selector 0x0c yields a zero byte) */
    const u32 schi03 = (sc03 >> 3) & 0x07070707u, sclo03 = sc03 & 0x07070707u;
    const u32 schi47 = (sc47 >> 3) & 0x07070707u, sclo47 = sc47 & 0x07070707u;
    auto pair_of_byte = [](u32 w, int k) { return __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (u32)k | ((u32)k << 16)); };

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

    ckq_v16i aH[2], aL[2];
    const ckq_v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    ckq_v8bf bm;
    ckq_v4i ab[2];
    float dxl = 0.0f;     /* block scale of the token of output (lane & 15) of this lane's 16-lane row */
    ckq_v16f i2;
    auto combine = [&](int ts, int r) {
        const int i1 = (aH[ts][r] << 3) + aL[ts][r];
        const float f = (float)i1;
        const float u = dw * f - dmin * i2[r];
        acc[ts][r] = fmac_row_lane(acc[ts][r], dxl, u, r);
        if constexpr (DUMP) {
            const int tok = 32 * ts + 8 * (r >> 2) + (r & 3);
            dl.put(tok, 0, i1);
            dl.put(tok, 1, (int)i2[r]);
        }
    };
    /* lane i of every 16-lane row fetches the scale of the token of its output r = i (through the
     * integer type: an LDS read of a float after a global->LDS load makes the compiler wait for that
     * load); the multiply-add of output r then takes lane r of the row as its factor */
    const int dx_tok = mfma32_row_of_lane(col + 32 * half);
    auto load_dx = [&](int ts) {
        dxl = __builtin_bit_cast(float, *reinterpret_cast<const int *>(&st.d[32 * ts + dx_tok]));
    };
    auto min_mfma = [&](int ts) {
        ckq_v16f zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.0f;
        i2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(ckq_v8bf, ab[ts]), bm, zero, 0, 0, 0);
    };

    CKQ_PIN();
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        const int ts = step_ts(s), j = step_j(s);
        if (s + 2 < 16) av[(s + 2) % 3] = a_read(s + 2);
        /* the first step of each token half starts from a literal zero accumulator */
        aH[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s % 3], bH[j], (s == 0 || s == 4) ? zero16 : aH[ts], 0, 0, 0);
        CKQ_PIN();     /* the MFMA first: VALU work that reads the previous MFMAs' results would otherwise wait in front of it */
        /* VALU work placed under this step's two MFMAs */
        if (s < 3) decode(s + 1);                    /* pass 1: planes 1..3 */
        else if (s >= 4 && s < 8) decode(s);         /* pass 2: planes 4..7 */
        else if (s == 8) {                           /* pass 3: min operands, scales of tokens 0-31 */
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
            ab[0] = lds16(reinterpret_cast<const uint8_t *>(&st.b[(col) * 16 + 8 * half]));
            ab[1] = lds16(reinterpret_cast<const uint8_t *>(&st.b[(32 + col) * 16 + 8 * half]));
        } else if (s == 10) load_dx(0);
        else if (s >= 12) { combine(0, 4 * (s - 12)); combine(0, 4 * (s - 12) + 1); }
        CKQ_PIN();
        aL[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s % 3], bL[j], (s == 0 || s == 4) ? zero16 : aL[ts], 0, 0, 0);
        if (s < 9) copy_one(s);                      /* one global->LDS copy of the next block per step */
        if (s == 11) min_mfma(0);                    /* tokens 0-31 are complete after this step */
        if (s >= 12) { combine(0, 4 * (s - 12) + 2); combine(0, 4 * (s - 12) + 3); }
        if (s == 15) asm volatile("" : "+v"(acc[0]));   /* the combine of tokens 0-31 stays under pass 4 */
        CKQ_PIN();
    }
    min_mfma(1);
    load_dx(1);
#pragma unroll
    for (int r = 0; r < 16; ++r) combine(1, r);
    asm volatile("" : "+v"(acc[1]));
#undef CKQ_PIN
}

/* KG = 2: the block is two groups of four waves on the same tile; group g takes
 * the K-blocks b0+g, b0+g+2, ... through its own pair of LDS stages, and the two
 * partial tiles are added through LDS at the end (group 0 + group 1, a fixed
 * order).  One such block fills a CU (two waves per SIMD) with ONE tile, so a
 * grid of T tiles takes ceil(T / 256) rounds of half-length tiles instead of
 * ceil(T / 512) rounds of full-length ones: 688 tiles need 3 x 0.5 instead of
 * 2 x 1. */
template <int WPE, int KG, bool DUMP = false>
__global__ void __launch_bounds__(256 * KG, KG == 2 ? 1 : WPE) gemm_q4k_mfma_kernel(GemmArgs a)
{
    constexpr int BM = GEMM_BM;
    __shared__ __attribute__((aligned(16))) GemmStage stage_all[KG][2];

    const int wave_all = wave_in_block();
    const int grp = KG == 2 ? wave_all >> 2 : 0, wave = wave_all & 3;
    const int tid = threadIdx.x & 255, lane = tid & 63;
    const int col = lane & 31, half = lane >> 5;
    GemmStage *const stage = stage_all[grp];

    const GemmWork work = gemm_work(a, a.nb);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * GEMM_BN;
    const u32 wstride = (u32)a.nb * 144u, xstride = (u32)a.nb * 292u;
    const int b0 = work.k0, b1 = work.k1, last = b1 - 1;
    const uint8_t *wbase = work.B + (size_t)n0 * wstride;       /* uniform */
    const uint8_t *xbase = a.A + (size_t)t0 * xstride;       /* uniform */

    /* Copy roles.  One wave instruction moves 64 x 16 bytes into 1 KiB of
     * LDS (lane l lands at byte 16 l).  Weights: the tile's 128 blocks of 144
     * bytes are 1152 chunks = 18 instructions, lane -> (row, ninth of the
     * block), so 9 consecutive lanes read one block contiguously.  Quants: 4
     * tokens per instruction, 16 lanes per token, the chunk order within a
     * token XOR-swizzled by the token number. */
    constexpr int NWI = 5, NQI = BM / 16;      /* per wave: 5 weight + 4 quant copies */
    u32 wofs_g[NWI], qofs_g[NQI];
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
        const int chunk = min(wave + 4 * i, 17) * 64 + lane, row = min(chunk / 9, work.N - 1 - n0), part = chunk % 9;
        wofs_g[i] = (u32)row * wstride + 16u * part;
    }
#pragma unroll
    for (int i = 0; i < NQI; ++i) {
        const int tl = 4 * (wave + 4 * i) + (lane >> 4), c = (lane & 15) ^ (tl & 15);
        qofs_g[i] = (u32)min(tl, a.M - 1 - t0) * xstride + 4u + 16u * c;
    }
    const int st_tok = tid >> 2, st_q = tid & 3;
    const bool st_live = st_tok < BM;
    const uint8_t *st_src = xbase + (size_t)min(st_tok, a.M - 1 - t0) * xstride;
    u32 nbs[2];
    float nd = 0.f;

    /* copies of block b into stage buf: the side loads (into registers) first,
     * then nine global->LDS instructions that copy_one(i) issues one at a
     * time so they can be spread over the MFMA steps */
    /* the copies address their source as buffer (uniform base in SGPRs) + per-lane
     * 32-bit offset + uniform K offset: no address arithmetic in the loop */
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_w = 0, cp_x = 0;
    int cp_buf = 0;
    auto copy_begin = [&](int b, int buf) {
        ld8<4>(nbs, st_src + (u32)b * 292u + 260 + 8 * st_q);
        nd = __builtin_bit_cast(float, ld4<4>(st_src + (u32)b * 292u));
        cp_w = b * 144;
        cp_x = b * 292;
        cp_buf = buf;
    };
    auto copy_one = [&](int i) {
        if (i < NWI)      /* weight slots past 17 repeat slot 17: same bytes, no branch */
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(stage[cp_buf].w + 1024 * min(wave + 4 * i, 17)), 16,
                                                     (int)wofs_g[i], cp_w, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].q + 1024 * (wave + 4 * (i - NWI))), 16,
                                                     (int)qofs_g[i - NWI], cp_x, 0, 0);
    };
    static_assert(NWI + NQI == 9, "the pipelined block issues nine copies");
    auto side_store = [&](int buf) {
        if (!st_live) return;
        if (st_q == 0) stage[buf].d[st_tok] = nd;
        const int b0 = (int)(int16_t)(nbs[0] & 0xffff) + (int)(int16_t)(nbs[0] >> 16);
        const int b1 = (int)(int16_t)(nbs[1] & 0xffff) + (int)(int16_t)(nbs[1] >> 16);
        u32 *bd = reinterpret_cast<u32 *>(&stage[buf].b[st_tok * 16]);
        bd[st_q]     = bf16_pair((float)(b0 & 63), (float)(b1 & 63));
        bd[4 + st_q] = bf16_pair((float)(64 * (b0 >> 6)), (float)(64 * (b1 >> 6)));
    };

    /* read-side offsets of this lane */
    const u32 wofs_l = (u32)(32 * wave + col) * 144u;   /* wave w owns rows 32w..32w+31 */
    u32 aofs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) aofs[j] = (u32)col * 256u + 16u * (u32)((2 * j + half) ^ (col & 15));

    ckq_v16f acc[2];
#pragma unroll
    for (int ts = 0; ts < 2; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ts][r] = 0.0f;

    copy_begin(min(b0 + grp, last), 0);
#pragma unroll
    for (int i = 0; i < NWI + NQI; ++i) copy_one(i);
    side_store(0);
    __builtin_amdgcn_s_waitcnt(0x0070);   /* vmcnt(0): this wave's copies have landed */
    __syncthreads();

    /* both groups run the same number of iterations (the barrier is the
     * block's); a group without a block in the last one only keeps step */
    const int niter = (b1 - b0 + KG - 1) / KG;
    /* One K-block.  The stage it reads is a compile-time constant (the loop
     * below is unrolled by the two stages), so every LDS address of the block is
     * a per-lane register set up once plus an immediate offset. */
    auto kstep = [&](int it, auto curc) {
        constexpr int cur = decltype(curc)::value;
        const int b = b0 + grp + KG * it;
        copy_begin(min(b + KG, last), cur ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        GemmDumpLane dl = {};
        if constexpr (DUMP) {
            const int n = n0 + wave * 32 + col, tf = t0 + 4 * half;
            dl.tok_stride = gemm_opaque((size_t)work.N * a.nb * 2);
            dl.p = a.dump + ((size_t)tf * work.N + n) * a.nb * 2 + (size_t)b * 2;
            dl.tok_left = a.M - tf;
            dl.row_ok = n < work.N && b < b1;
        }
        if (KG == 1 || b < b1) gemm_block_pipe<DUMP>(stage[cur], wofs_l, aofs, col, half, acc, copy_one, dl);
        __builtin_amdgcn_sched_barrier(0);
        side_store(cur ^ 1);
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();
    };
    for (int it = 0; it < niter; it += 2) {
        kstep(it, std::integral_constant<int, 0>{});
        if (it + 1 < niter) kstep(it + 1, std::integral_constant<int, 1>{});
    }

    if constexpr (KG == 2) {
        /* partial tile of group 1 through LDS (every stage is idle now) */
        float *red = reinterpret_cast<float *>(&stage_all[0][0]);
        static_assert(sizeof(GemmStage) >= 32 * 256 * sizeof(float), "the reduction buffer fits one stage");
        if (grp == 1) {
#pragma unroll
            for (int ts = 0; ts < 2; ++ts)
#pragma unroll
                for (int r = 0; r < 16; ++r) red[(ts * 16 + r) * 256 + tid] = acc[ts][r];
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int ts = 0; ts < 2; ++ts)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ts][r] += red[(ts * 16 + r) * 256 + tid];
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

/* Which token tile a launch takes.  A 96-token tile (ckq_gemm_q4k_t96.hip) costs 1.37 times a 64-token one for 1.5
 * times the tokens, in blocks that run that much longer and leave a 32- or 64-token remainder tile that costs 0.6 / 0.8 of
 * a whole one: it pays when every block has a CU to itself, when one round of its blocks replaces a round and a bit of
 * 64-token tiles, or when the grid is at least a round and a half deep; it loses when a few long blocks are left over for
 * a second round (512 tokens x 11008 rows: 516 blocks on 512 slots, 67 us against 62) and when CUs that hold two of its
 * blocks compete with 64-token tiles that all fit one round (960 x 4096: 52.6 against 45.4).  `tiles64`: tiles of the 64-token kernel, `blocks96`: blocks of the 96-token one. */
static std::atomic<int> g_q4k_tile{0};
extern "C" void ckq_launch_set_q4k_tile(int tokens) { g_q4k_tile.store(tokens == 64 || tokens == 96 ? tokens : 0); }
static bool q4k_take_t96(int M, int tiles64, int blocks96)
{
    const int forced = g_q4k_tile.load(std::memory_order_relaxed);
    if (forced) return forced == 96;
    constexpr int SLOTS = 512;                /* 256 CUs, two blocks each */
    if (M < 576 || tiles64 <= 256) return false;
    if (blocks96 <= SLOTS / 2) return true;                  /* every block has a CU to itself: 36 us against 40 */
    if (blocks96 <= SLOTS) return tiles64 > SLOTS;           /* one round, against a second round of 64-token tiles */
    return 2 * blocks96 >= 3 * SLOTS;
}

int launch_gemm_q4k_mfma(const void *A, const void *B, const float *bias, float *C,
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
    if ((long long)g.nb * 292 * GEMM_BN >= (1ll << 31)) return (int)hipErrorInvalidValue;
    g.ntt = (M + GEMM_BM - 1) / GEMM_BM;
    g.nnt = (N + GEMM_BN - 1) / GEMM_BN;
    const int nnt8 = (g.nnt + 7) / 8 * 8;
    /* One tile per CU at most (with the K split the launch will choose) and a
     * long enough K: two groups of waves per tile put a second wave on every
     * SIMD (4096x11008 at M = 512: 80 -> 70 us).  With more tiles than CUs two
     * independent blocks per CU interleave better than two groups in lockstep
     * (11008x4096: 78 us against 88). */
    const int tiles = g.ntt * g.nnt, sp = gemm_choose_splits(tiles, g.nb);
    const bool two_groups = tiles * sp <= 256 && (g.nb + sp - 1) / sp >= 8;
    if (q4k_take_t96(M, tiles, gemm_q4k_t96_token_tiles(M) * g.nnt)) return launch_gemm_q4k_t96(g, s);
    if (sums) {
#if CKQ_WITH_DUMP
        if (two_groups) return gemm_launch_split(gemm_q4k_mfma_kernel<CKQ_GEMM_WPE, 2, true>, g, (unsigned)(g.ntt * nnt8), g.nb, s, 512);
        return gemm_launch_split(gemm_q4k_mfma_kernel<CKQ_GEMM_WPE, 1, true>, g, (unsigned)(g.ntt * nnt8), g.nb, s, 256);
#else
        return CKQ_ENODUMP;
#endif
    }
    if (two_groups) return gemm_launch_split(gemm_q4k_mfma_kernel<CKQ_GEMM_WPE, 2>, g, (unsigned)(g.ntt * nnt8), g.nb, s, 512);
    return gemm_launch_split(gemm_q4k_mfma_kernel<CKQ_GEMM_WPE, 1>, g, (unsigned)(g.ntt * nnt8), g.nb, s, 256);
}

int launch_gemm_q4k_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s)
{
    const int tiles = gemm_group_tiles(in, M, GEMM_BM);
    if (tiles < GEMM_GROUP_MIN_TILES) return CKQ_ENOGROUP;
    GemmArgs g = {};
    g.A = (const uint8_t *)A; g.M = M; g.nb = K / 256;
    if ((long long)g.nb * 292 * GEMM_BN >= (1ll << 31)) return (int)hipErrorInvalidValue;
    if (q4k_take_t96(M, tiles, gemm_group_tiles(in, M, 96))) return launch_gemm_q4k_t96_group(g, in, s);
    g.ntt = (M + GEMM_BM - 1) / GEMM_BM;
    /* as for one matrix: two groups of waves per tile while every tile gets a CU of its own */
    if (tiles <= 256 && g.nb >= 8) return gemm_launch_grouped(gemm_q4k_mfma_kernel<CKQ_GEMM_WPE, 2>, g, in, s, 512);
    return gemm_launch_grouped(gemm_q4k_mfma_kernel<CKQ_GEMM_WPE, 1>, g, in, s, 256);
}
