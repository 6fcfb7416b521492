/*
 * ckq_formats.hpp - per-format traits for the dequant-dot kernels.
 *
 * A weight row is cut into "positions": the unit of work of one lane.
 *   Q4_K / Q5_K : one 64-element group of a super-block (header + 32 B of
 *                 nibbles [+ 32 B of fifth bits]); two sub-blocks, two scales.
 *   Q6_K        : 64 elements of a super-block: a 16-wide slice l0 of one
 *                 128-half, i.e. elements l0+{0,32,64,96}+[0,16); 48 B of
 *                 quants, four scales.
 *   Q8_0        : one 32-element block (34 B).
 * Each trait provides
 *   Off / w_off    byte offsets of the position inside a weight row, computed
 *                  once per lane (loads are then uniform row base + 32-bit offset),
 *   Wt  / load_w   raw weight dwords of a position (nothing decoded yet, so all
 *                  loads of a wave can be in flight together),
 *   Act / load_act the activation slice the position multiplies with,
 *   Dec / decode   quants unpacked to int8x4 dwords and integer scales,
 *   dot            integer sub-block dots -> integer block-scale combination
 *                  -> one fp32 partial,
 *   NSUB / dump    the raw integer sub-block dots, for the bit-exactness tests.
 *
 * Arithmetic contracts (reference file:line):
 *   Q4_K x Q8_K  gemm_kernels_q4k_q8k.c:121-181   d*sc*S - dmin*m*(stored bsums)
 *   Q5_K x Q8_K  gemm_kernels_q5_k.c:130-208      same with 5-bit quants
 *   Q6_K x Q8_K  gemm_kernels_q6k_q8k.c:601-695   d * sum_s sc_s*sum (q-32)*q8, bsums unused
 *   Q8_0 x Q8_0  gemm_kernels_q8_0.c:968-989      sumi * (fp16 dw * fp16 dx)
 *   Q8_0 x fp32  gemm_kernels_q8_0.c:254-277      sum d*q*x
 */
#pragma once
#include "ckq_device.hpp"

/* 6-bit scale/min pair of sub-blocks (2g, 2g+1) from the 12 packed bytes
 * (layout: reference include/ckernel_quant.h:227-251).  u0,u1,u2 are the
 * three little-endian words of scales[12].  Returns sc in the low two bytes
 * of *sc2 (byte 0 = sub-block 2g) and likewise the mins. */
__device__ __forceinline__ void k4_scale_pair(u32 u0, u32 u1, u32 u2, int g, u32 *sc2, u32 *mn2)
{
    const int sh = 16 * (g & 1);
    const u32 a = u0 >> sh, b = u1 >> sh, c = u2 >> sh;
    const u32 sc_lo = a & 0x3f3fu, mn_lo = b & 0x3f3fu;
    const u32 sc_hi = (c & 0x0f0fu) | (((a >> 6) & 0x0303u) << 4);
    const u32 mn_hi = ((c >> 4) & 0x0f0fu) | (((b >> 6) & 0x0303u) << 4);
    *sc2 = g < 2 ? sc_lo : sc_hi;
    *mn2 = g < 2 ? mn_lo : mn_hi;
}

/* ------------------------------------------------------------------------- */
struct FmtQ4K {
    static constexpr int POS_PER_BLOCK = 4, WBLOCK = 144, XBLOCK = 292, NSUB = 2;
    static constexpr int OCC1 = 8, OCC2 = 6;   /* waves per SIMD the one-token kernel is held to: one row, two rows per wave */
    static constexpr bool TOKEN_TILES = true; /* tiles of 2, 4 and 8 tokens exist */
    struct Wt  { u32 hdr[4]; u32 qs[8]; };
    struct Act { int q[16]; float d; int b_lo, b_hi; };
    struct Dec { int lo[8], hi[8]; int sc_lo, sc_hi, mn_lo, mn_hi; float d, dmin; };

    struct Off { u32 hdr, qs; };   /* byte offsets inside a weight row */
    static __device__ __forceinline__ Off w_off(int pos)
    {
        Off o;
        o.hdr = (u32)(pos >> 2) * WBLOCK;
        o.qs  = o.hdr + 16 + 32 * (pos & 3);
        return o;
    }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { o.hdr += s; o.qs += s; }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o)
    {
        ld16<4>(w.hdr, row + o.hdr);
        ld16<4>(w.qs, row + o.qs);
        ld16<4>(w.qs + 4, row + o.qs + 16);
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const uint8_t *blk = x + (u32)(pos >> 2) * XBLOCK;
        const int g = pos & 3;
        a.d = __builtin_bit_cast(float, ld4<4>(blk));
        for (int i = 0; i < 4; ++i) ld16<4>(a.q + 4 * i, blk + 4 + 64 * g + 16 * i);
        u32 bs[2];
        ld8<4>(bs, blk + 260 + 8 * g);   /* stored bsums[4g..4g+3] */
        a.b_lo = (int)(int16_t)(bs[0] & 0xffff) + (int)(int16_t)(bs[0] >> 16);
        a.b_hi = (int)(int16_t)(bs[1] & 0xffff) + (int)(int16_t)(bs[1] >> 16);
    }
    /* Staging of the token tile's activation rows in LDS: units of XS_SRC
     * source bytes travel through XS_REGS registers; here the LDS image is a
     * plain copy. */
    static constexpr int XS_SRC = 16, XS_REGS = 4;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return tile_bytes; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p) { ld16<XBLOCK % 4 == 0 ? 4 : 2>(v, p); }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 16u * unit);
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int tl, int pos, u32 xrow, int, u32)
    {
        load_act(a, xs + (u32)tl * xrow, pos);
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int pos)
    {
        u32 sc2, mn2;
        k4_scale_pair(w.hdr[1], w.hdr[2], w.hdr[3], pos & 3, &sc2, &mn2);
        d.sc_lo = sc2 & 0xff; d.sc_hi = (sc2 >> 8) & 0xff;
        d.mn_lo = mn2 & 0xff; d.mn_hi = (mn2 >> 8) & 0xff;
        d.d = h2f(w.hdr[0] & 0xffff);
        d.dmin = h2f(w.hdr[0] >> 16);
        for (int i = 0; i < 8; ++i) {
            d.lo[i] = (int)(w.qs[i] & 0x0f0f0f0fu);
            d.hi[i] = (int)((w.qs[i] >> 4) & 0x0f0f0f0fu);
        }
    }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        int s_lo = 0, s_hi = 0;
        for (int i = 0; i < 8; ++i) {
            s_lo = dot4(d.lo[i], a.q[i], s_lo);
            s_hi = dot4(d.hi[i], a.q[8 + i], s_hi);
        }
        sub[0] = s_lo; sub[1] = s_hi;
        const int i1 = mul24(d.sc_lo, s_lo) + mul24(d.sc_hi, s_hi);
        const int i2 = mul24(d.mn_lo, a.b_lo) + mul24(d.mn_hi, a.b_hi);
        return (d.d * a.d) * (float)i1 - (d.dmin * a.d) * (float)i2;
    }
    /* index of sub[i] among the 8 sub-block dots of the position's block */
    static __device__ __forceinline__ int sub_index(int pos, int i) { return 8 * (pos >> 2) + 2 * (pos & 3) + i; }
    static constexpr int SUBS_PER_BLOCK = 8;
};

/* ------------------------------------------------------------------------- */
struct FmtQ5K {
    static constexpr int POS_PER_BLOCK = 4, WBLOCK = 176, XBLOCK = 292, NSUB = 2;
    static constexpr int OCC1 = 8, OCC2 = 5;            /* waves per SIMD the one-token kernel is held to */
    static constexpr bool TOKEN_TILES = true; /* tiles of 2, 4 and 8 tokens exist */
    struct Wt  { u32 hdr[4]; u32 qh[8]; u32 qs[8]; };
    typedef FmtQ4K::Act Act;
    typedef FmtQ4K::Dec Dec;

    typedef FmtQ4K::Off Off;
    static __device__ __forceinline__ Off w_off(int pos)
    {
        Off o;
        o.hdr = (u32)(pos >> 2) * WBLOCK;
        o.qs  = o.hdr + 48 + 32 * (pos & 3);
        return o;
    }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { o.hdr += s; o.qs += s; }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o)
    {
        ld16<4>(w.hdr, row + o.hdr);
        ld16<4>(w.qh, row + o.hdr + 16);
        ld16<4>(w.qh + 4, row + o.hdr + 32);
        ld16<4>(w.qs, row + o.qs);
        ld16<4>(w.qs + 4, row + o.qs + 16);
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos) { FmtQ4K::load_act(a, x, pos); }
    /* Staging of the token tile's activation rows in LDS: units of XS_SRC
     * source bytes travel through XS_REGS registers; here the LDS image is a
     * plain copy. */
    static constexpr int XS_SRC = 16, XS_REGS = 4;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return tile_bytes; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p) { ld16<XBLOCK % 4 == 0 ? 4 : 2>(v, p); }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 16u * unit);
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int tl, int pos, u32 xrow, int, u32)
    {
        load_act(a, xs + (u32)tl * xrow, pos);
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int pos)
    {
        const int g = pos & 3;
        u32 sc2, mn2;
        k4_scale_pair(w.hdr[1], w.hdr[2], w.hdr[3], g, &sc2, &mn2);
        d.sc_lo = sc2 & 0xff; d.sc_hi = (sc2 >> 8) & 0xff;
        d.mn_lo = mn2 & 0xff; d.mn_hi = (mn2 >> 8) & 0xff;
        d.d = h2f(w.hdr[0] & 0xffff);
        d.dmin = h2f(w.hdr[0] >> 16);
        for (int i = 0; i < 8; ++i) {
            const u32 h = w.qh[i] >> (2 * g);   /* bit 0: fifth bit of low-nibble element, bit 1: of high-nibble element */
            d.lo[i] = (int)((w.qs[i] & 0x0f0f0f0fu) | ((h & 0x01010101u) << 4));
            d.hi[i] = (int)(((w.qs[i] >> 4) & 0x0f0f0f0fu) | (((h >> 1) & 0x01010101u) << 4));
        }
    }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub) { return FmtQ4K::dot(d, a, sub); }
    static __device__ __forceinline__ int sub_index(int pos, int i) { return FmtQ4K::sub_index(pos, i); }
    static constexpr int SUBS_PER_BLOCK = 8;
};

/* ------------------------------------------------------------------------- */
struct FmtQ6K {
    static constexpr int POS_PER_BLOCK = 4, WBLOCK = 210, XBLOCK = 292, NSUB = 4;
    static constexpr int OCC1 = 8, OCC2 = 6;   /* waves per SIMD the one-token kernel is held to: one row, two rows per wave */
    static constexpr bool TOKEN_TILES = true; /* tiles of 2, 4 and 8 tokens exist */
    struct Wt  { u32 ql0[4], ql1[4], qh[4]; u32 sc[2]; u32 d; };
    struct Act { int q[16]; float d; int a32[4]; };      /* a32[r] = 32 * sum of the run's 16 quants */
    struct Dec { int q[16]; int sc[4]; float d; };

    struct Off { u32 ql, qh, sc, d; };
    static __device__ __forceinline__ Off w_off(int pos)
    {
        const u32 blk = (u32)(pos >> 2) * WBLOCK;
        const int n = (pos >> 1) & 1, l0 = 16 * (pos & 1);
        Off o;
        o.ql = blk + 64 * n + l0;
        o.qh = blk + 128 + 32 * n + l0;
        o.sc = blk + 192 + 8 * n;
        o.d  = blk + 208;
        return o;
    }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { o.ql += s; o.qh += s; o.sc += s; o.d += s; }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o)
    {
        ld16<2>(w.ql0, row + o.ql);
        ld16<2>(w.ql1, row + o.ql + 32);
        ld16<2>(w.qh, row + o.qh);
        ld8<2>(w.sc, row + o.sc);
        w.d = ld2(row + o.d);
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const uint8_t *blk = x + (u32)(pos >> 2) * XBLOCK;
        const int n = (pos >> 1) & 1, l0 = 16 * (pos & 1);
        a.d = __builtin_bit_cast(float, ld4<4>(blk));
        for (int r = 0; r < 4; ++r) {
            ld16<4>(a.q + 4 * r, blk + 4 + 128 * n + 32 * r + l0);
            int s = 0;
            for (int i = 0; i < 4; ++i) s = dot4(0x01010101, a.q[4 * r + i], s);
            a.a32[r] = 32 * s;   /* computed from the quants: the reference's x86 routine never reads bsums here */
        }
    }
    /* Staging of the token tile's activation rows in LDS: units of XS_SRC
     * source bytes travel through XS_REGS registers; here the LDS image is a
     * plain copy. */
    static constexpr int XS_SRC = 16, XS_REGS = 4;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return tile_bytes; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p) { ld16<XBLOCK % 4 == 0 ? 4 : 2>(v, p); }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 16u * unit);
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int tl, int pos, u32 xrow, int, u32)
    {
        load_act(a, xs + (u32)tl * xrow, pos);
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int pos)
    {
        const int odd = pos & 1;
        for (int i = 0; i < 4; ++i) {
            const u32 h = w.qh[i];
            d.q[i]      = (int)((w.ql0[i] & 0x0f0f0f0fu)        | ((h & 0x03030303u) << 4));
            d.q[4 + i]  = (int)((w.ql1[i] & 0x0f0f0f0fu)        | (((h >> 2) & 0x03030303u) << 4));
            d.q[8 + i]  = (int)(((w.ql0[i] >> 4) & 0x0f0f0f0fu) | (((h >> 4) & 0x03030303u) << 4));
            d.q[12 + i] = (int)(((w.ql1[i] >> 4) & 0x0f0f0f0fu) | (((h >> 6) & 0x03030303u) << 4));
        }
        /* scales[8n + odd + 2r], r = 0..3 */
        d.sc[0] = sbyte(w.sc[0], odd);
        d.sc[1] = sbyte(w.sc[0], odd + 2);
        d.sc[2] = sbyte(w.sc[1], odd);
        d.sc[3] = sbyte(w.sc[1], odd + 2);
        d.d = h2f(w.d);
    }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        int i1 = 0;
        for (int r = 0; r < 4; ++r) {
            int s = 0;
            for (int i = 0; i < 4; ++i) s = dot4(d.q[4 * r + i], a.q[4 * r + i], s);
            s -= a.a32[r];              /* sum (q-32)*q8 = sum q*q8 - 32*sum q8 */
            sub[r] = s;
            i1 += mul24(d.sc[r], s);
        }
        return (d.d * a.d) * (float)i1;
    }
    static __device__ __forceinline__ int sub_index(int pos, int r)
    {
        return 16 * (pos >> 2) + 8 * ((pos >> 1) & 1) + (pos & 1) + 2 * r;
    }
    static constexpr int SUBS_PER_BLOCK = 16;
};

/* ------------------------------------------------------------------------- */
struct FmtQ80 {
    static constexpr int POS_PER_BLOCK = 1, WBLOCK = 34, XBLOCK = 34, NSUB = 1;
    static constexpr int OCC1 = 8, OCC2 = 6;   /* waves per SIMD the one-token kernel is held to: one row, two rows per wave */
    static constexpr bool TOKEN_TILES = true; /* tiles of 2, 4 and 8 tokens exist */
    struct Wt  { u32 q[8]; u32 d; };
    struct Act { int q[8]; float d; };
    struct Dec { int q[8]; float d; };

    struct Off { u32 blk; };
    static __device__ __forceinline__ Off w_off(int pos)
    {
        Off o;
        o.blk = (u32)pos * WBLOCK;
        return o;
    }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { o.blk += s; }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o)
    {
        w.d = ld2(row + o.blk);
        ld16<2>(w.q, row + o.blk + 2);
        ld16<2>(w.q + 4, row + o.blk + 18);
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const uint8_t *blk = x + (u32)pos * XBLOCK;
        a.d = h2f(ld2(blk));
        ld16<2>(a.q, blk + 2);
        ld16<2>(a.q + 4, blk + 18);
    }
    /* Staging of the token tile's activation rows in LDS.  A 34-byte block at a
     * 2-byte aligned address makes every 16-byte LDS read misaligned, so the
     * tile is re-laid out: the quants of block j at byte 32 j, its scale as
     * fp32 at 32 * total + 4 j. */
    static constexpr int XS_SRC = 34, XS_REGS = 9;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return tile_bytes / 34 * 36; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p)
    {
        v[8] = ld2(p);
        ld16<2>(v, p + 2);
        ld16<2>(v + 4, p + 18);
    }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32 total)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 32u * unit);
        for (int i = 0; i < 8; ++i) d[i] = v[i];
        *reinterpret_cast<float *>(xs + 32u * total + 4u * unit) = h2f(v[8]);
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int tl, int pos, u32, int npos, u32 total)
    {
        const u32 j = (u32)tl * (u32)npos + (u32)pos;
        const u32 *q = reinterpret_cast<const u32 *>(xs + 32u * j);
        for (int i = 0; i < 8; ++i) a.q[i] = (int)q[i];
        a.d = *reinterpret_cast<const float *>(xs + 32u * total + 4u * j);
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int)
    {
        for (int i = 0; i < 8; ++i) d.q[i] = (int)w.q[i];
        d.d = h2f(w.d);
    }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        int s = 0;
        for (int i = 0; i < 8; ++i) s = dot4(d.q[i], a.q[i], s);
        sub[0] = s;
        return (float)s * (d.d * a.d);
    }
    static __device__ __forceinline__ int sub_index(int pos, int) { return pos; }
    static constexpr int SUBS_PER_BLOCK = 1;
};

/* Q8_0 rows of an even number of blocks, taken two blocks (68 bytes) per
 * position.  A 34-byte block starts 2 bytes off a dword boundary in every
 * second block, and 16-byte loads at such addresses run 14 % below the aligned
 * rate; a pair starts on a dword boundary (row pitch 34 * even), so its 17
 * dwords are loaded aligned and the first block's quants, which sit 2 bytes in,
 * are realigned in registers with v_alignbyte (the second block's quants start
 * at byte 36 and need nothing).  Same integer dots; a lane adds its two blocks'
 * fp32 terms before the cross-lane sum. */
struct FmtQ80P : FmtQ80 {
    static constexpr int NSUB = 2;
    static constexpr int OCC1 = 6, OCC2 = 4;   /* 17 weight + 18 activation registers per position */
    struct Wt  { u32 v[17]; };
    struct Act { int q[16]; float d[2]; };
    struct Dec { int q[16]; float d[2]; };
    static __device__ __forceinline__ Off w_off(int pos)
    {
        Off o;
        o.blk = (u32)pos * 68u;
        return o;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o)
    {
        const uint8_t *p = row + o.blk;
        ld16<4>(w.v, p);
        ld16<4>(w.v + 4, p + 16);
        ld16<4>(w.v + 8, p + 32);
        ld16<4>(w.v + 12, p + 48);
        w.v[16] = ld4<4>(p + 64);
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const uint8_t *blk = x + (u32)pos * 68u;
        a.d[0] = h2f(ld2(blk));
        ld16<2>(a.q, blk + 2);
        ld16<2>(a.q + 4, blk + 18);
        a.d[1] = h2f(ld2(blk + 34));
        ld16<2>(a.q + 8, blk + 36);
        ld16<2>(a.q + 12, blk + 52);
    }
    /* the staged image is FmtQ80's (per 34-byte block); a position reads two consecutive blocks */
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int tl, int pos, u32, int npos, u32 total)
    {
        const u32 j = 2u * ((u32)tl * (u32)npos + (u32)pos);
        const u32 *q = reinterpret_cast<const u32 *>(xs + 32u * j);
        for (int i = 0; i < 16; ++i) a.q[i] = (int)q[i];
        const float *d = reinterpret_cast<const float *>(xs + 32u * total + 4u * j);
        a.d[0] = d[0];
        a.d[1] = d[1];
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int)
    {
        d.d[0] = h2f(w.v[0] & 0xffffu);
        for (int i = 0; i < 8; ++i) d.q[i] = (int)__builtin_amdgcn_alignbyte(w.v[i + 1], w.v[i], 2);
        d.d[1] = h2f(w.v[8] >> 16);
        for (int i = 0; i < 8; ++i) d.q[8 + i] = (int)w.v[9 + i];
    }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        int s0 = 0, s1 = 0;
        for (int i = 0; i < 8; ++i) s0 = dot4(d.q[i], a.q[i], s0);
        for (int i = 0; i < 8; ++i) s1 = dot4(d.q[8 + i], a.q[8 + i], s1);
        sub[0] = s0;
        sub[1] = s1;
        return (float)s0 * (d.d[0] * a.d[0]) + (float)s1 * (d.d[1] * a.d[1]);
    }
    static __device__ __forceinline__ int sub_index(int pos, int r) { return 2 * pos + r; }
};

/* Q5_0 weights against Q8_0 activations: 22-byte blocks (fp16 d, 32 fifth bits,
 * 16 nibble bytes), values q - 16 in [-16, 15]; everything on the activation
 * side is FmtQ80's.  Reference: gemm_kernels_q5_0.c:901-939. */
struct FmtQ50 : FmtQ80 {
    static constexpr int WBLOCK = 22;
    struct Wt { u32 qs[4]; u32 qh; u32 d; };
    static __device__ __forceinline__ Off w_off(int pos)
    {
        Off o;
        o.blk = (u32)pos * WBLOCK;
        return o;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o)
    {
        w.d = ld2(row + o.blk);
        w.qh = ld4<2>(row + o.blk + 2);
        ld16<2>(w.qs, row + o.blk + 6);
    }
    /* four 5-bit values (nibbles in n, their fifth bits in the low four bits
     * of h) minus 16, as packed int8 */
    static __device__ __forceinline__ int q5_bytes(u32 n, u32 h)
    {
        const u32 spread = ((h & 15u) * 0x00204081u) & 0x01010101u;      /* bit k -> byte k */
        const u32 v = n | (spread << 4);                                  /* 0..31 per byte */
        return (int)((((v | 0x80808080u) - 0x10101010u)) ^ 0x80808080u);  /* - 16 per byte, no borrows */
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int)
    {
        for (int i = 0; i < 4; ++i) {
            d.q[i]     = q5_bytes(w.qs[i] & 0x0f0f0f0fu, w.qh >> (4 * i));
            d.q[4 + i] = q5_bytes((w.qs[i] >> 4) & 0x0f0f0f0fu, w.qh >> (16 + 4 * i));
        }
        d.d = h2f(w.d);
    }
};

/* Q8_0 weights against fp32 activations (no activation quantization). */
struct FmtQ80F32 {
    static constexpr int POS_PER_BLOCK = 1, WBLOCK = 34, XBLOCK = 128, NSUB = 1;
    static constexpr int OCC1 = 4, OCC2 = 1;            /* 64 activation floats per lane: 128 registers */
    static constexpr bool TOKEN_TILES = false;
    typedef FmtQ80::Wt Wt;
    typedef FmtQ80::Dec Dec;
    struct Act { float x[32]; };

    typedef FmtQ80::Off Off;
    static __device__ __forceinline__ Off w_off(int pos) { return FmtQ80::w_off(pos); }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { FmtQ80::off_shift(o, s); }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o) { FmtQ80::load_w(w, row, o); }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const uint8_t *p = x + (u32)pos * XBLOCK;
        for (int i = 0; i < 8; ++i) {
            u32 t[4];
            ld16<4>(t, p + 16 * i);
            for (int j = 0; j < 4; ++j) a.x[4 * i + j] = __builtin_bit_cast(float, t[j]);
        }
    }
    /* A lane reads a run of consecutive 16-byte units; lanes are 128 bytes
     * apart, so unswizzled they would all hit the same LDS banks. */
    static __device__ __forceinline__ u32 xs_unit(u32 u) { return u ^ ((u >> 4) & 15u); }
    static constexpr int XS_SRC = 16, XS_REGS = 4;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return (tile_bytes + 255) & ~(size_t)255; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p) { ld16<4>(v, p); }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 16u * xs_unit(unit));
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int, int pos, u32, int, u32)
    {
        for (int i = 0; i < 8; ++i) {
            u32 t[4];
            ld16<4>(t, xs + 16u * xs_unit(8u * (u32)pos + i));
            for (int j = 0; j < 4; ++j) a.x[4 * i + j] = __builtin_bit_cast(float, t[j]);
        }
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int pos) { FmtQ80::decode(d, w, pos); }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        float s = 0.0f;
        for (int i = 0; i < 8; ++i)
            for (int j = 0; j < 4; ++j) s += (d.d * (float)sbyte((u32)d.q[i], j)) * a.x[4 * i + j];
        sub[0] = 0;
        return s;
    }
    static __device__ __forceinline__ int sub_index(int pos, int) { return pos; }
    static constexpr int SUBS_PER_BLOCK = 1;
};

/* Q4_K weights against fp32 activations (no activation quantization):
 * sum (d*sc*q - dmin*m) * x (reference: gemm_kernels_q4k.c:53-101). */
struct FmtQ4KF32 {
    static constexpr int POS_PER_BLOCK = 4, WBLOCK = 144, XBLOCK = 1024, NSUB = 1;
    static constexpr int OCC1 = 4, OCC2 = 1;            /* 64 activation floats per lane: 128 registers */
    static constexpr bool TOKEN_TILES = false;
    typedef FmtQ4K::Wt Wt;
    typedef FmtQ4K::Dec Dec;
    struct Act { float x[64]; };

    typedef FmtQ4K::Off Off;
    static __device__ __forceinline__ Off w_off(int pos) { return FmtQ4K::w_off(pos); }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { FmtQ4K::off_shift(o, s); }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o) { FmtQ4K::load_w(w, row, o); }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const uint8_t *p = x + (u32)pos * 256u;      /* 64 floats per position */
        for (int i = 0; i < 16; ++i) {
            u32 t[4];
            ld16<4>(t, p + 16 * i);
            for (int j = 0; j < 4; ++j) a.x[4 * i + j] = __builtin_bit_cast(float, t[j]);
        }
    }
    /* lanes are 256 bytes apart: swizzle the unit index so 16 lanes reading
     * their i-th unit touch 16 different bank groups */
    static __device__ __forceinline__ u32 xs_unit(u32 u) { return u ^ ((u >> 4) & 15u); }
    static constexpr int XS_SRC = 16, XS_REGS = 4;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return (tile_bytes + 255) & ~(size_t)255; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p) { ld16<4>(v, p); }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 16u * xs_unit(unit));
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int, int pos, u32, int, u32)
    {
        for (int i = 0; i < 16; ++i) {
            u32 t[4];
            ld16<4>(t, xs + 16u * xs_unit(16u * (u32)pos + i));
            for (int j = 0; j < 4; ++j) a.x[4 * i + j] = __builtin_bit_cast(float, t[j]);
        }
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int pos) { FmtQ4K::decode(d, w, pos); }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        const float d1 = d.d * (float)d.sc_lo, m1 = d.dmin * (float)d.mn_lo;
        const float d2 = d.d * (float)d.sc_hi, m2 = d.dmin * (float)d.mn_hi;
        float s = 0.0f;
        for (int i = 0; i < 8; ++i)
            for (int j = 0; j < 4; ++j) {
                s += (d1 * (float)((d.lo[i] >> (8 * j)) & 0xff) - m1) * a.x[4 * i + j];
                s += (d2 * (float)((d.hi[i] >> (8 * j)) & 0xff) - m2) * a.x[32 + 4 * i + j];
            }
        sub[0] = 0;
        return s;
    }
    static __device__ __forceinline__ int sub_index(int pos, int) { return pos; }
    static constexpr int SUBS_PER_BLOCK = 4;
};

/* Q6_K weights against fp32 activations: sum (d*sc*(q-32)) * x
 * (reference: gemm_kernels_q6k.c:39-76). */
struct FmtQ6KF32 {
    static constexpr int POS_PER_BLOCK = 4, WBLOCK = 210, XBLOCK = 1024, NSUB = 1;
    static constexpr int OCC1 = 4, OCC2 = 1;            /* 64 activation floats per lane: 128 registers */
    static constexpr bool TOKEN_TILES = false;
    typedef FmtQ6K::Wt Wt;
    typedef FmtQ6K::Dec Dec;
    struct Act { float x[64]; };                     /* four runs of 16: elements 128n + 32r + 16*odd + i */

    typedef FmtQ6K::Off Off;
    static __device__ __forceinline__ Off w_off(int pos) { return FmtQ6K::w_off(pos); }
    static __device__ __forceinline__ void off_shift(Off &o, u32 s) { FmtQ6K::off_shift(o, s); }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, const Off &o) { FmtQ6K::load_w(w, row, o); }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *x, int pos)
    {
        const int n = (pos >> 1) & 1, l0 = 16 * (pos & 1);
        const uint8_t *blk = x + (u32)(pos >> 2) * 1024u + 4u * (u32)(128 * n + l0);
        for (int r = 0; r < 4; ++r)
            for (int i = 0; i < 4; ++i) {
                u32 t[4];
                ld16<4>(t, blk + 128 * r + 16 * i);
                for (int j = 0; j < 4; ++j) a.x[16 * r + 4 * i + j] = __builtin_bit_cast(float, t[j]);
            }
    }
    static __device__ __forceinline__ u32 xs_unit(u32 u) { return u ^ ((u >> 4) & 15u); }
    static constexpr int XS_SRC = 16, XS_REGS = 4;
    static __host__ __device__ __forceinline__ size_t xs_lds_bytes(size_t tile_bytes) { return (tile_bytes + 255) & ~(size_t)255; }
    static __device__ __forceinline__ void xs_ld(u32 (&v)[XS_REGS], const uint8_t *p) { ld16<4>(v, p); }
    static __device__ __forceinline__ void xs_st(uint8_t *xs, const u32 (&v)[XS_REGS], u32 unit, u32)
    {
        u32 *d = reinterpret_cast<u32 *>(xs + 16u * xs_unit(unit));
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
    static __device__ __forceinline__ void load_act_lds(Act &a, const uint8_t *xs, int, int pos, u32, int, u32)
    {
        const int n = (pos >> 1) & 1, l0 = 16 * (pos & 1);
        const u32 u0 = 64u * (u32)(pos >> 2) + (u32)(128 * n + l0) / 4u;      /* unit of the first float */
        for (int r = 0; r < 4; ++r)
            for (int i = 0; i < 4; ++i) {
                u32 t[4];
                ld16<4>(t, xs + 16u * xs_unit(u0 + 8u * r + i));
                for (int j = 0; j < 4; ++j) a.x[16 * r + 4 * i + j] = __builtin_bit_cast(float, t[j]);
            }
    }
    static __device__ __forceinline__ void decode(Dec &d, const Wt &w, int pos) { FmtQ6K::decode(d, w, pos); }
    static __device__ __forceinline__ float dot(const Dec &d, const Act &a, int *sub)
    {
        float s = 0.0f;
        for (int r = 0; r < 4; ++r) {
            const float ds = d.d * (float)d.sc[r];
            for (int i = 0; i < 4; ++i)
                for (int j = 0; j < 4; ++j)
                    s += (ds * (float)(((d.q[4 * r + i] >> (8 * j)) & 0xff) - 32)) * a.x[16 * r + 4 * i + j];
        }
        sub[0] = 0;
        return s;
    }
    static __device__ __forceinline__ int sub_index(int pos, int) { return pos; }
    static constexpr int SUBS_PER_BLOCK = 4;
};
