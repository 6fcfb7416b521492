/* ckq_pure.c - see ckq_pure.h. */
#include "ckq_pure.h"

#include <stdlib.h>
#include <string.h>
#include <strings.h>

uint64_t ckq_fingerprint(const void *p, size_t bytes)
{
    /* FNV-1a-style mixing over 64 samples of 64 bytes spread across the range, eight bytes at a
     * time (a byte-wise hash of the same 4 KB costs 3.5 us of every host-pointer call) */
    const uint8_t *b = (const uint8_t *)p;
    uint64_t h = 0xcbf29ce484222325ull ^ bytes;
    const size_t chunk = 64, n = 64;
    const size_t step = bytes > chunk * n ? (bytes - chunk) / (n - 1) : chunk;
    for (size_t i = 0; i < n; ++i) {
        size_t off = i * step;
        if (off >= bytes) break;
        size_t len = bytes - off < chunk ? bytes - off : chunk, j = 0;
        for (; j + 8 <= len; j += 8) {
            uint64_t w;
            memcpy(&w, b + off + j, 8);
            h = (h ^ w) * 0x100000001b3ull;
            h ^= h >> 29;
        }
        for (; j < len; ++j) h = (h ^ b[off + j]) * 0x100000001b3ull;
    }
    return h;
}

int ckq_ranges_overlap(const void *a, size_t na, const void *b, size_t nb)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a0 < b0 + nb && b0 < a0 + na;
}

int ckq_split_rows(int M, int ith, int nth, int whole, int *r0, int *r1)
{
    if (M <= 0 || ith < 0 || nth <= 0 || ith >= nth) return 0;
    if (whole) {
        if (ith != 0) return 0;
        *r0 = 0;
        *r1 = M;
        return 1;
    }
    const int dr = (int)(((long)M + nth - 1) / nth);
    const long lo = (long)dr * ith;
    if (lo >= M) return 0;
    *r0 = (int)lo;
    *r1 = lo + dr < M ? (int)(lo + dr) : M;
    return 1;
}

void ckq_grid_chunk(long total, long per, long c, long *first, long *count)
{
    *first = c * per;
    *count = total - *first < per ? total - *first : per;
    if (*count < 0) *count = 0;
}

int ckq_workspace_pick(const uint64_t *keys, const uint64_t *last_use, int n, uint64_t key)
{
    int free_slot = -1, lru = 0;
    for (int i = 0; i < n; ++i) {
        if (keys[i] == key) return i;
        if (keys[i] == 0 && free_slot < 0) free_slot = i;
        if (last_use[i] < last_use[lru]) lru = i;
    }
    return free_slot >= 0 ? free_slot : lru;
}

int ckq_manifest_parse_line(char *line, unsigned long long *size, unsigned long long *runtime_offset)
{
    static const char *const quant[] = {"q4_k", "q4k", "q5_k", "q5k", "q6_k", "q6k", "q8_0", "q80", "q5_0", "q50"};
    char *p = line;
    while (*p == ' ' || *p == '\t') ++p;
    if (*p == '#' || *p == '\n' || *p == '\r' || *p == 0) return 0;
    char *f[5];
    int nf = 0;
    for (char *q = p; nf < 5; ++nf) {
        f[nf] = q;
        char *bar = strchr(q, '|');
        if (!bar) { ++nf; break; }
        *bar = 0;
        q = bar + 1;
    }
    if (nf < 5) return -1;
    int is_quant = 0;
    for (size_t i = 0; i < sizeof quant / sizeof quant[0]; ++i) is_quant |= strcasecmp(f[1], quant[i]) == 0;
    if (!is_quant) return 0;
    *size = strtoull(f[3], NULL, 0);
    *runtime_offset = strtoull(f[4], NULL, 0);
    return *size != 0;
}
