/*
 * ckq_gemm_q6k.hip - prefill GEMM, Q6_K weights x Q8_K activations, on the
 * gfx950 int8 matrix cores.
 *
 *   C[t][n] = sum_b (dw(n,b) * dx(t,b)) * (float) I(t,n,b)   (+ bias[n])
 *   I = sum_{s<16} sc(n,b,s) * sum_{k in 16-run s} (q6(n,k) - 32) * q8(t,k)     (exact int32)
 * which is the per-block arithmetic of the reference's x86 dot product
 * (gemm_kernels_q6k_q8k.c:601-695: integer sum per block, one fp32 scale per
 * block) under its token loop (gemm_kernels_q6k_q8k.c:1243-1268).
 *
 * Mapping to the hardware
 * - v_mfma_i32_32x32x32_i8 takes 32 k per instruction; a lane supplies the 16 k
 *   of one half, which is exactly one 16-run of a Q6_K block, so every lane
 *   works with ONE int8 scale per instruction.
 * - The scaled weight v = sc * (q6 - 32) needs 14 bits.  It is formed once per
 *   weight in 16-bit lanes (v_pk_mad_u16 on byte pairs) and split into two int8
 *   planes v = 256 * H + L, L = the signed low byte of v, H = the high byte of
 *   v + 128; both planes are accumulated over the whole 256-block and
 *   I = 256 * IH + IL exactly.  The split costs nothing: the two planes are the
 *   byte lanes of the 16-bit products, gathered with v_perm_b32.
 * - Operands reach LDS by 16-byte global->LDS loads.  A 210-byte block is
 *   fetched as 14 chunks; the last one starts at byte 194 so that no load
 *   reaches past the block (it carries the fp16 scale in its last two bytes).
 *   Rows are only 2-byte aligned in memory; the loads accept that.  Quants
 *   are laid out as in the Q4_K kernel (chunks XOR-swizzled by token).
 * - Block = 4 waves = (32 * TH tokens) x 128 weight rows, wave w owns rows
 *   32w..32w+31 and all TH token groups of 32.  The kernel is bound by VALU
 *   issue (about 11 operations per 4 weights against one MFMA per 512 weight
 *   bytes), so plane expansion of k-slab s+1 is interleaved with the MFMAs of
 *   slab s and larger token tiles (TH = 4) amortise it where the grid is big
 *   enough to fill the chip with them.
 */
#include "ckq_gemm_common.hpp"
#include <atomic>
#include <type_traits>

constexpr int GEMM6_BN  = 128;   /* weight rows per tile */
constexpr int GEMM6_ROW = 224;   /* LDS bytes per staged weight block: 14 chunks */

template <int TH> struct Gemm6Stage {
    uint8_t w[GEMM6_BN * GEMM6_ROW];   /* row r at 224 r: chunks 0-12 = block bytes 0..207, chunk 13 = bytes 194..209 */
    uint8_t q[32 * TH * 256];          /* int8 quants: 16-byte chunk c of token t in slot c ^ (t & 15) of its 256 bytes */
    float   d[32 * TH];                /* block scale of each token */
};


/* What a lane reads from a stage before it can start on a block: its row's
 * raw Q6_K block (the 16-byte runs its k-half touches) and the activation
 * operands of the first k-slab.  Read right after the barrier that publishes
 * the stage, ahead of the previous block's fp32 combine, which hides the LDS
 * latency. */
template <int TH> struct Gemm6Head {
    ckq_v4i ql[2][2], qh[2], scv, av0[TH];
    u32 dw16;
};

template <int TH>
__device__ __forceinline__ void gemm6_head_read(const uint8_t *w, const uint8_t *q, u32 wrow, u32 aofs0, int half, Gemm6Head<TH> &h)
{
    auto lds16 = [&](const uint8_t *p) { return *reinterpret_cast<const ckq_v4i *>(p); };
    const uint8_t *wr = w + wrow;
#pragma unroll
    for (int n = 0; n < 2; ++n) {
#pragma unroll
        for (int odd = 0; odd < 2; ++odd) h.ql[n][odd] = lds16(wr + 16 * (4 * n + 2 * odd + half));
        h.qh[n] = lds16(wr + 16 * (8 + 2 * n + half));
    }
    h.scv = lds16(wr + 192);
    h.dw16 = *reinterpret_cast<const uint16_t *>(wr + 222);
#pragma unroll
    for (int ts = 0; ts < TH; ++ts) h.av0[ts] = lds16(&q[aofs0 + 32 * 256 * ts]);
}

/* Integer sums of one block and the scales they are combined under. */
template <int TH> struct Gemm6Sums {
    ckq_v16i iL[TH], iH[TH];
    float    dx[TH];     /* per token group: the block scale of the token of output (lane & 15) */
    float    dw;
};

template <int TH, bool DUMP>
__device__ __forceinline__ void gemm6_combine(const Gemm6Sums<TH> &p, ckq_v16f (&acc)[TH], const GemmDumpLane &dl)
{
#pragma unroll
    for (int ts = 0; ts < TH; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i = (p.iH[ts][r] << 8) + p.iL[ts][r];
            acc[ts][r] = fmac_row_lane(acc[ts][r], p.dx[ts], p.dw * (float)i, r);
            if constexpr (DUMP) dl.put(32 * ts + 8 * (r >> 2) + (r & 3), 0, i);
        }
}

/* The integer part of one 256-block of a tile: eight k-slabs of 32, each 2*TH
 * MFMAs (TH token groups x two planes).  The planes of slab s+1 are expanded
 * between the MFMAs of slab s; copy_one(i) issues one global->LDS copy of a
 * later block. */
template <int TH, int NCOPY, class CopyFn>
__device__ __forceinline__ void gemm6_slabs(const uint8_t *q, const float *d, const Gemm6Head<TH> &h, const u32 (&aofs)[8], int half,
                                            Gemm6Sums<TH> &out, CopyFn copy_one)
{
#define CKQ_PIN() __builtin_amdgcn_sched_barrier(0)
    auto lds16 = [&](const uint8_t *p) { return *reinterpret_cast<const ckq_v4i *>(p); };
    const int sh0 = 8 * half, sh1 = 16 + 8 * half;   /* scale of slab s: byte 2 (s & 1) + half of dword s >> 1 */

    ckq_v4i av[2][TH];
#pragma unroll
    for (int ts = 0; ts < TH; ++ts) av[0][ts] = h.av0[ts];
    auto a_read = [&](int s) {
#pragma unroll
        for (int ts = 0; ts < TH; ++ts) av[s & 1][ts] = lds16(&q[aofs[s] + 32 * 256 * ts]);
    };

    /* token scales: read before the first copy is issued (an LDS read of a
     * float after a global->LDS load would wait for the load), and through the
     * integer vector type like every other read of a stage */
    const int dx_tok = mfma32_row_of_lane((int)(threadIdx.x & 63));
#pragma unroll
    for (int ts = 0; ts < TH; ++ts)
        out.dx[ts] = __builtin_bit_cast(float, *reinterpret_cast<const int *>(&d[32 * ts + dx_tok]));
    out.dw = h2f(h.dw16);

    u32 scp[2], cp[2];
    ckq_v4i pL[2], pH[2];
    auto prep = [&](int s) {
        const int sc = __builtin_amdgcn_sbfe(h.scv[s >> 1], (s & 1) ? sh1 : sh0, 8);
        scp[s & 1] = __builtin_amdgcn_perm((u32)sc, (u32)sc, 0x05040504u);          /* sc in both 16-bit lanes */
        cp[s & 1]  = pk_mad_u16(scp[s & 1], 0xFFE0FFE0u, 0x00800080u);              /* 128 - 32 sc */
    };
    auto decode = [&](int s, int i) {
        const int n = s >> 2, g = s & 3;
        const u32 lw = (u32)h.ql[n][g & 1][i], hw = (u32)h.qh[n][i];
        const u32 nib = g < 2 ? (lw & 0x0f0f0f0fu) : ((lw >> 4) & 0x0f0f0f0fu);
        const u32 hb = g == 0 ? (hw << 4) : g == 1 ? (hw << 2) : g == 2 ? hw : (hw >> 2);
        const u32 q = (hb & 0x30303030u) | nib;                                   /* four 6-bit values */
        const u32 e = __builtin_amdgcn_perm(0u, q, 0x0c020c00u);                  /* bytes 0, 2 in 16-bit lanes */
        const u32 o = __builtin_amdgcn_perm(0u, q, 0x0c030c01u);                  /* bytes 1, 3 */
        const u32 te = pk_mad_u16(e, scp[s & 1], cp[s & 1]);                      /* sc * (q - 32) + 128 */
        const u32 to = pk_mad_u16(o, scp[s & 1], cp[s & 1]);
        pL[s & 1][i] = (int)(__builtin_amdgcn_perm(to, te, 0x06020400u) ^ 0x80808080u);
        pH[s & 1][i] = (int)__builtin_amdgcn_perm(to, te, 0x07030501u);
    };

    const ckq_v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    prep(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) decode(0, i);
    CKQ_PIN();
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        if (s < 7) prep(s + 1);
#pragma unroll
        for (int k = 0; k < 2 * TH; ++k) {
            const int ts = k >> 1;
            if ((k & 1) == 0) out.iL[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s & 1][ts], pL[s & 1], s == 0 ? zero16 : out.iL[ts], 0, 0, 0);
            else              out.iH[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[s & 1][ts], pH[s & 1], s == 0 ? zero16 : out.iH[ts], 0, 0, 0);
            /* VALU work under this MFMA: a share of the next slab's planes */
            if (s < 7) {
                constexpr int PER = TH >= 4 ? 2 : 1;           /* MFMAs per decoded dword */
                if (k % PER == 0 && k / PER < 4) decode(s + 1, k / PER);
            }
            if (k == 0 && s < 7) a_read(s + 1);       /* operands of the next slab, three MFMAs ahead of their use */
            /* copies of a later block, spread over the slabs */
            if ((k & 1) == 0 && s + 4 * k < NCOPY) copy_one(s + 4 * k);
            CKQ_PIN();
        }
    }
#undef CKQ_PIN
}

template <int TH, bool DUMP = false>
__global__ void __launch_bounds__(256, 1) gemm_q6k_mfma_kernel(GemmArgs a)
{
    constexpr int BM = 32 * TH;
    /* Blocks are fetched NST-1 iterations ahead.  The weights stream from HBM
     * and a fetch takes about as long as one iteration of a 64-token tile, so
     * that tile runs three stages deep (136 KB of LDS); the 128-token tile has
     * room for two. */
    constexpr int NST = TH == 2 ? 3 : 2;
    __shared__ __attribute__((aligned(16))) Gemm6Stage<TH> stage[NST];

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int col = lane & 31, half = lane >> 5;

    /* token tiles fastest inside an XCD, so each XCD's L2 sees a weight tile once */
    const GemmWork work = gemm_work(a, a.nb);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * GEMM6_BN;
    const u32 wstride = (u32)a.nb * 210u, xstride = (u32)a.nb * 292u;
    const int b0 = work.k0, b1 = work.k1, last = b1 - 1;
    const uint8_t *wbase = work.B + (size_t)n0 * wstride;       /* uniform */
    const uint8_t *xbase = a.A + (size_t)t0 * xstride;       /* uniform */

    /* Copy roles.  One wave instruction moves 64 x 16 bytes into 1 KiB of LDS
     * (lane l lands at byte 16 l).  Weights: 128 rows x 14 chunks = 28
     * instructions, seven per wave.  Quants: 4 tokens per instruction. */
    constexpr int NWI = 7, NQI = BM / 16, NDI = BM / 64, NCOPY = NWI + NQI + NDI;
    static_assert(NCOPY <= 8 * TH, "one copy per pair of MFMAs at most");
    u32 wofs_g[NWI], qofs_g[NQI], dofs_g[NDI];
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
        const int chunk = (wave + 4 * i) * 64 + lane, row = min(chunk / 14, work.N - 1 - n0), part = chunk % 14;
        wofs_g[i] = (u32)row * wstride + (part < 13 ? 16u * part : 194u);
    }
#pragma unroll
    for (int i = 0; i < NQI; ++i) {
        const int tl = 4 * (wave + 4 * i) + (lane >> 4), c = (lane & 15) ^ (tl & 15);
        qofs_g[i] = (u32)min(tl, a.M - 1 - t0) * xstride + 4u + 16u * c;
    }
    /* token scales: 4-byte copies, lane l fetches the scale of token 64 i + l.
     * Every wave issues them (same bytes to the same place), which keeps the
     * number of outstanding copies equal in all waves. */
#pragma unroll
    for (int i = 0; i < NDI; ++i) dofs_g[i] = (u32)min(64 * i + lane, a.M - 1 - t0) * xstride;

    /* the copies address their source as buffer (uniform base in SGPRs) + per-lane
     * 32-bit offset + uniform K offset: no address arithmetic in the loop */
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_w = 0, cp_x = 0;
    int cp_buf = 0;
    auto copy_begin = [&](int b, int buf) {
        cp_w = b * 210;
        cp_x = b * 292;
        cp_buf = buf;
    };
    auto copy_one = [&](int i) {
        if (i < NWI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(stage[cp_buf].w + 1024 * (wave + 4 * i)), 16, (int)(wofs_g[i]), cp_w, 0, 0);
        else if (i < NWI + NQI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].q + 1024 * (wave + 4 * (i - NWI))), 16,
                                                     (int)qofs_g[i - NWI], cp_x, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(stage[cp_buf].d + 64 * (i - NWI - NQI)), 4, (int)(dofs_g[i - NWI - NQI]), cp_x, 0, 0);
    };

    /* read-side offsets of this lane */
    const u32 wrow = (u32)(32 * wave + col) * (u32)GEMM6_ROW;
    u32 aofs[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) aofs[s] = (u32)col * 256u + 16u * (u32)((2 * s + half) ^ (col & 15));

    ckq_v16f acc[TH];
#pragma unroll
    for (int ts = 0; ts < TH; ++ts)
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

    /* The loop holds no other memory operation than the copies, so the wait
     * before the barrier counts them exactly: block b+1 has landed when only
     * the copies issued during this iteration (three stages) or none (two) are
     * still in flight.  A bare s_barrier: the block's waves exchange data only
     * through those copies. */
    Gemm6Head<TH> head;
    gemm6_head_read<TH>(stage[0].w, stage[0].q, wrow, aofs[0], half, head);
    /* One K-block.  With three stages the stage it reads (and the one it fills)
     * is a compile-time constant - the loop below is unrolled over the stages -
     * so the LDS addresses of a block are per-lane registers set up once plus
     * immediates. */
    auto kstep = [&](int b, auto curc) {
        const int cur = curc, pf = cur == 0 ? NST - 1 : cur - 1, nxt = cur + 1 == NST ? 0 : cur + 1;
        copy_begin(min(b + NST - 1, last), pf);
        __builtin_amdgcn_sched_barrier(0);
        Gemm6Sums<TH> sums;
        GemmDumpLane dl = {};
        if constexpr (DUMP) {
            const int n = n0 + wave * 32 + col, tf = t0 + 4 * half;
            dl.tok_stride = gemm_opaque((size_t)work.N * a.nb);
            dl.p = a.dump + ((size_t)tf * work.N + n) * a.nb + (size_t)b;
            dl.tok_left = a.M - tf;
            dl.row_ok = n < work.N;
        }
        gemm6_slabs<TH, NCOPY>(stage[cur].q, stage[cur].d, head, aofs, half, sums, copy_one);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NST == 3) __builtin_amdgcn_s_waitcnt(0x0070 | (NCOPY & 15) | ((NCOPY >> 4) << 14));
        else                    __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        /* The next block's first reads, then this block's fp32 combine under
         * them (after the last block the stage holds that block again: unused).
         * The 128-token tile has no registers to spare for that overlap. */
        if constexpr (TH == 2) {
            gemm6_head_read<TH>(stage[nxt].w, stage[nxt].q, wrow, aofs[0], half, head);
            __builtin_amdgcn_sched_barrier(0);
            gemm6_combine<TH, DUMP>(sums, acc, dl);
        } else {
            gemm6_combine<TH, DUMP>(sums, acc, dl);
            __builtin_amdgcn_sched_barrier(0);
            gemm6_head_read<TH>(stage[nxt].w, stage[nxt].q, wrow, aofs[0], half, head);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (NST == 3) {
        for (int b = b0; b < b1; b += 3) {
            kstep(b, std::integral_constant<int, 0>{});
            if (b + 1 < b1) kstep(b + 1, std::integral_constant<int, 1>{});
            if (b + 2 < b1) kstep(b + 2, std::integral_constant<int, 2>{});
        }
    } else {            /* the 128-token tile has no registers to spare for constant-stage addressing */
        int cur = 0;
        for (int b = b0; b < b1; ++b, cur ^= 1) kstep(b, cur);
    }

    const GemmOut o = work.out;
    const int n = n0 + wave * 32 + col;
    if (n < work.N) {
        const float bias = o.bias ? o.bias[n] : 0.0f;
#pragma unroll
        for (int ts = 0; ts < TH; ++ts)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * ts + 8 * (r >> 2) + 4 * half + (r & 3);
                if (t < a.M) gemm_store(&o.C[(size_t)t * o.ldc + n], acc[ts][r] + bias);
            }
    }
}

/* Two blocks per CU: the 64-token tile with ONE LDS image of the weights and two of the activations (60.5 KB).
 * A lane takes its row's whole raw block into registers at the start of a 256-block (gemm6_head_read), so a
 * barrier behind those reads frees the image for the next block's weights; a second, independent block on
 * the CU fills the waits this shallower pipeline leaves (a fetch has one iteration to land instead of two)
 * and lets one wave's MFMAs run under the other's plane expansion.  Every LDS region is an object of its own:
 * the compiler then puts no wait for a copy in front of the reads of another region. */
template <int TH, bool DUMP = false>
__global__ void __launch_bounds__(256, 2) gemm_q6k_pair_kernel(GemmArgs a)
{
    constexpr int BM = 32 * TH;
    __shared__ __attribute__((aligned(16))) uint8_t wimg[GEMM6_BN * GEMM6_ROW];
    __shared__ __attribute__((aligned(16))) uint8_t q_even[BM * 256], q_odd[BM * 256];
    __shared__ __attribute__((aligned(16))) float d_even[(BM + 63) / 64 * 64], d_odd[(BM + 63) / 64 * 64];
    auto qst = [&](auto c) __attribute__((always_inline)) -> uint8_t * { if constexpr (decltype(c)::value == 0) return q_even; else return q_odd; };
    auto dst = [&](auto c) __attribute__((always_inline)) -> float * { if constexpr (decltype(c)::value == 0) return d_even; else return d_odd; };

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int col = lane & 31, half = lane >> 5;

    const GemmWork work = gemm_work(a, a.nb);
    const int id = work.id, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= work.nnt) return;
    const int t0 = tt * BM, n0 = nt * GEMM6_BN;
    const u32 wstride = (u32)a.nb * 210u, xstride = (u32)a.nb * 292u;
    const int b0 = work.k0, b1 = work.k1, last = b1 - 1;
    const uint8_t *wbase = work.B + (size_t)n0 * wstride;
    const uint8_t *xbase = a.A + (size_t)t0 * xstride;

    /* copy roles as in gemm_q6k_mfma_kernel<2> */
    constexpr int NWI = 7, NQI = BM / 16, NDI = (BM + 63) / 64, NCOPY = NWI + NQI + NDI;
    u32 wofs_g[NWI], qofs_g[NQI], dofs_g[NDI];
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
        const int chunk = (wave + 4 * i) * 64 + lane, row = min(chunk / 14, work.N - 1 - n0), part = chunk % 14;
        wofs_g[i] = (u32)row * wstride + (part < 13 ? 16u * part : 194u);
    }
#pragma unroll
    for (int i = 0; i < NQI; ++i) {
        const int tl = 4 * (wave + 4 * i) + (lane >> 4), c = (lane & 15) ^ (tl & 15);
        qofs_g[i] = (u32)min(tl, a.M - 1 - t0) * xstride + 4u + 16u * c;
    }
#pragma unroll
    for (int i = 0; i < NDI; ++i) dofs_g[i] = (u32)min(64 * i + lane, a.M - 1 - t0) * xstride;
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void *)wbase, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)xbase, 0, 0x7fffffff, 0x00020000);
    int cp_w = 0, cp_x = 0;
    auto copy_begin = [&](int b) __attribute__((always_inline)) {
        cp_w = b * 210;
        cp_x = b * 292;
    };
    auto copy_one = [&](int i, auto bufc) __attribute__((always_inline)) {
        if (i < NWI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (ckq_lds_void *)(wimg + 1024 * (wave + 4 * i)), 16, (int)(wofs_g[i]), cp_w, 0, 0);
        else if (i < NWI + NQI)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(qst(bufc) + 1024 * (wave + 4 * (i - NWI))), 16,
                                                     (int)qofs_g[i - NWI], cp_x, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (ckq_lds_void *)(dst(bufc) + 64 * (i - NWI - NQI)), 4, (int)dofs_g[i - NWI - NQI], cp_x, 0, 0);
    };

    const u32 wrow = (u32)(32 * wave + col) * (u32)GEMM6_ROW;
    u32 aofs[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) aofs[s] = (u32)col * 256u + 16u * (u32)((2 * s + half) ^ (col & 15));

    ckq_v16f acc[TH];
#pragma unroll
    for (int ts = 0; ts < TH; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ts][r] = 0.0f;

    copy_begin(b0);
#pragma unroll
    for (int i = 0; i < NCOPY; ++i) copy_one(i, std::integral_constant<int, 0>{});
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();

    Gemm6Head<TH> head;
    gemm6_head_read<TH>(wimg, q_even, wrow, aofs[0], half, head);
    auto kstep = [&](int b, auto curc) __attribute__((always_inline)) {
        constexpr int cur = decltype(curc)::value;
        /* every wave has its rows of the weight image in registers: the image takes the next block */
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        copy_begin(min(b + 1, last));
        __builtin_amdgcn_sched_barrier(0);
        Gemm6Sums<TH> sums;
        GemmDumpLane dl = {};
        if constexpr (DUMP) {
            const int n = n0 + wave * 32 + col, tf = t0 + 4 * half;
            dl.tok_stride = gemm_opaque((size_t)work.N * a.nb);
            dl.p = a.dump + ((size_t)tf * work.N + n) * a.nb + (size_t)b;
            dl.tok_left = a.M - tf;
            dl.row_ok = n < work.N;
        }
        auto copy_next = [&](int i) __attribute__((always_inline)) { copy_one(i, std::integral_constant<int, cur ^ 1>{}); };
        gemm6_slabs<TH, NCOPY>(qst(curc), dst(curc), head, aofs, half, sums, copy_next);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        /* the next block's first reads, then this block's fp32 combine under them */
        gemm6_head_read<TH>(wimg, qst(std::integral_constant<int, cur ^ 1>{}), wrow, aofs[0], half, head);
        __builtin_amdgcn_sched_barrier(0);
        gemm6_combine<TH, DUMP>(sums, acc, dl);
        __builtin_amdgcn_sched_barrier(0);
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
        for (int ts = 0; ts < TH; ++ts)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * ts + 8 * (r >> 2) + 4 * half + (r & 3);
                if (t < a.M) gemm_store(&o.C[(size_t)t * o.ldc + n], acc[ts][r] + bias);
            }
    }
}

/* Which launches take the paired kernel.  It spends 12 % more per token than the 128-token tiles at one block per CU
 * and about as much as the three-stage 64-token kernel, but its grid has 512 slots of 64 tokens instead of 256 of 128, and
 * a partly filled last round runs faster instead of costing a whole block time: it is taken when the 128-token grid
 * would waste a quarter or more of its last round (512 tokens x 11008 rows, K = 4096: 344 tiles on 256 CUs, 94.8 us;
 * paired 78.7) and there are at least 512 blocks of 64 tokens.  variant: 0 = by shape, 1 = never, 2 = always. */
static std::atomic<int> g_q6k_variant{0};
extern "C" void ckq_launch_set_q6k_variant(int variant) { g_q6k_variant.store(variant == 1 || variant == 2 ? variant : 0); }
static bool q6k_take_pair(int tiles128, int tiles64)
{
    const int forced = g_q6k_variant.load(std::memory_order_relaxed);
    if (forced) return forced == 2;
    if (tiles64 < 512 || tiles128 <= 256) return false;
    const int rounds = (tiles128 + 255) / 256;
    return 4 * rounds * 256 >= 5 * tiles128;        /* ceil(r) / r >= 1.25 */
}

int launch_gemm_q6k_mfma(const void *A, const void *B, const float *bias, float *C,
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
    g.nnt = (N + GEMM6_BN - 1) / GEMM6_BN;
    const int nnt8 = (g.nnt + 7) / 8 * 8;
    if (q6k_take_pair(((M + 127) / 128) * g.nnt, ((M + 63) / 64) * g.nnt)) {
        g.ntt = (M + 63) / 64;
#if CKQ_WITH_DUMP
        if (sums) return gemm_launch_split(gemm_q6k_pair_kernel<2, true>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
#else
        if (sums) return CKQ_ENODUMP;
#endif
        return gemm_launch_split(gemm_q6k_pair_kernel<2>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
    }
    /* tiles of 128 tokens where they still give every CU work, else 64 */
    const int ntt4 = (M + 127) / 128;
    if (ntt4 * g.nnt > 128) {
        g.ntt = ntt4;
#if CKQ_WITH_DUMP
        if (sums) return gemm_launch_split(gemm_q6k_mfma_kernel<4, true>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
#else
        if (sums) return CKQ_ENODUMP;
#endif
        return gemm_launch_split(gemm_q6k_mfma_kernel<4>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
    }
    g.ntt = (M + 63) / 64;
#if CKQ_WITH_DUMP
    if (sums) return gemm_launch_split(gemm_q6k_mfma_kernel<2, true>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
#else
    if (sums) return CKQ_ENODUMP;
#endif
    return gemm_launch_split(gemm_q6k_mfma_kernel<2>, g, (unsigned)(g.ntt * nnt8), g.nb, s);
}

int launch_gemm_q6k_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s)
{
    GemmArgs g = {};
    g.A = (const uint8_t *)A; g.M = M; g.nb = K / 256;
    if ((long long)g.nb * 292 * 128 >= (1ll << 31)) return (int)hipErrorInvalidValue;
    /* tiles of 128 tokens where they fill the chip, else 64 */
    if (gemm_group_tiles(in, M, 128) >= GEMM_GROUP_MIN_TILES) {
        g.ntt = (M + 127) / 128;
        return gemm_launch_grouped(gemm_q6k_mfma_kernel<4>, g, in, s);
    }
    if (gemm_group_tiles(in, M, 64) < GEMM_GROUP_MIN_TILES) return CKQ_ENOGROUP;
    g.ntt = (M + 63) / 64;
    return gemm_launch_grouped(gemm_q6k_mfma_kernel<2>, g, in, s);
}
