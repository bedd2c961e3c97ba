/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's host entropy codec for packed
 * ternary tensors (static 3-symbol range coder with a 16-bit PMF and bytewise renormalisation,
 * plus the 26-byte big-endian container). Nothing in the shipped package links this file.
 *
 * Restates (paths relative to the reference root):
 *   RangeEncoder / RangeDecoder          tmq/rangecoder.h:41-193
 *   WriteStream / ReadStream (byte use)  tmq/bitstream.h:31-177
 *   entropyEncodeTernary / Decode        tmq/tmq_native.cpp:50-140
 * Pinned by: byte-for-byte comparison with the compiled reference (oracle/_ref) in this
 * container, committed golden streams produced by it, and encode->decode round trips.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    uint8_t *buf;
    size_t len, cap;
} bytes_t;

static int put(bytes_t *b, uint8_t v) {
    if (b->len == b->cap) {
        size_t nc = b->cap ? b->cap * 2 : 4096;
        uint8_t *nb = (uint8_t *)realloc(b->buf, nc);
        if (!nb) return -1;
        b->buf = nb;
        b->cap = nc;
    }
    b->buf[b->len++] = v;
    return 0;
}

static void be64(uint8_t *p, uint64_t v) { for (int i = 0; i < 8; i++) p[i] = (uint8_t)(v >> (56 - 8 * i)); }
static void be32(uint8_t *p, uint32_t v) { for (int i = 0; i < 4; i++) p[i] = (uint8_t)(v >> (24 - 8 * i)); }
static void be16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)(v >> 8); p[1] = (uint8_t)v; }
static uint64_t rd64(const uint8_t *p) { uint64_t v = 0; for (int i = 0; i < 8; i++) v = (v << 8) | p[i]; return v; }
static uint32_t rd32(const uint8_t *p) { uint32_t v = 0; for (int i = 0; i < 4; i++) v = (v << 8) | p[i]; return v; }
static uint16_t rd16(const uint8_t *p) { return (uint16_t)((p[0] << 8) | p[1]); }

/* Renormalisation predicate shared by coder and decoder, tmq/rangecoder.h:77-78, 164-165:
 * emit while the top byte is settled, or -- on underflow -- after shrinking the range to the
 * distance to the next 64 Ki boundary.                                                       */
static inline int renorm_needed(uint32_t low, uint32_t *range) {
    if ((low ^ (low + *range)) < 0x01000000u) return 1;
    if (*range < 0x00010000u) {
        *range = (0u - low) & 0xFFFFu;
        return 1;
    }
    return 0;
}

/*
 * Encode packed words [rows][ceil(columns/16)] (only the first `columns` codes of each row are
 * symbols). Returns a malloc'd container in *out (caller frees with tmq_oracle_free) and its
 * size, or a negative code: -1 code 11 met, -2 a used symbol got probability 0 (the reference
 * would not terminate), -3 out of memory / too large.
 */
int64_t tmq_oracle_compress(const uint32_t *words, int64_t rows, int64_t columns, uint8_t **out) {
    static const uint8_t symtable[4] = {1, 2, 0, 3}; /* code -> symbol; symbols are -1, 0, +1 */
    int64_t histo[4] = {0, 0, 0, 0};
    int64_t qcols = (columns + 15) / 16;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t qc = 0; qc < qcols; qc++) {
            uint32_t w = words[r * qcols + qc];
            int lim = (int)((columns - qc * 16) < 16 ? (columns - qc * 16) : 16);
            for (int i = 0; i < lim; i++) histo[symtable[(w >> (2 * (15 - i))) & 3u]]++;
        }
    if (histo[3] != 0) return -1;
    int64_t total = histo[0] + histo[1] + histo[2];
    float scale = 65535.f / (float)total;
    uint16_t pmf[3];
    uint32_t cmf[3];
    for (int i = 0; i < 3; i++) pmf[i] = (uint16_t)((float)histo[i] * scale);
    cmf[0] = 0;
    cmf[1] = cmf[0] + pmf[0];
    cmf[2] = cmf[1] + pmf[1];
    uint32_t tot = cmf[2] + pmf[2];
    for (int i = 0; i < 3; i++)
        if (histo[i] > 0 && pmf[i] == 0) return -2;

    bytes_t bs = {0, 0, 0};
    uint32_t low = 0, range = 0xFFFFFFFFu;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t qc = 0; qc < qcols; qc++) {
            uint32_t w = words[r * qcols + qc];
            int lim = (int)((columns - qc * 16) < 16 ? (columns - qc * 16) : 16);
            for (int i = 0; i < lim; i++) {
                int s = symtable[(w >> (2 * (15 - i))) & 3u];
                range /= tot;
                low += cmf[s] * range;
                range *= pmf[s];
                while (renorm_needed(low, &range)) {
                    if (put(&bs, (uint8_t)(low >> 24))) { free(bs.buf); return -3; }
                    range <<= 8;
                    low <<= 8;
                }
            }
        }
    for (int i = 0; i < 4; i++) { /* flush, tmq/rangecoder.h:91-97 */
        if (put(&bs, (uint8_t)(low >> 24))) { free(bs.buf); return -3; }
        low <<= 8;
    }
    /* The byte stream of the reference always carries one trailing zero byte that is counted
     * in the size but not in the bit count (tmq/bitstream.h:33-36, 91-95). */
    size_t nbytes = bs.len + 1;
    uint64_t nbits = (uint64_t)bs.len * 8u;
    size_t totalsize = nbytes + 8 + 8 + 4 + 6;
    if (totalsize > 0xFFFFFFFFull) { free(bs.buf); return -3; }
    uint8_t *o = (uint8_t *)malloc(totalsize);
    if (!o) { free(bs.buf); return -3; }
    be64(o, (uint64_t)(rows * columns));
    be64(o + 8, nbits);
    be32(o + 16, (uint32_t)totalsize);
    for (int i = 0; i < 3; i++) be16(o + 20 + 2 * i, pmf[i]);
    if (bs.len) memcpy(o + 26, bs.buf, bs.len);
    o[26 + bs.len] = 0;
    free(bs.buf);
    *out = o;
    return (int64_t)totalsize;
}

void tmq_oracle_free(void *p) { free(p); }

/* Decode a container into packed words [rows][ceil(columns/16)]. Returns the symbol count
 * stored in the header, or a negative code for a malformed header.                           */
int64_t tmq_oracle_decompress(const uint8_t *in, int64_t in_size, uint32_t *words, int64_t rows,
                              int64_t columns) {
    static const uint8_t codetable[3] = {2, 0, 1}; /* symbol -> code */
    if (in_size < 26) return -1;
    uint64_t numsyms = rd64(in);
    if (numsyms == 0) { words[0] = 0; return 0; }
    uint64_t nbits = rd64(in + 8);
    uint32_t totalsize = rd32(in + 16);
    if (totalsize < 26) return -1;
    uint16_t pmf[3];
    uint32_t cmf[3];
    for (int i = 0; i < 3; i++) pmf[i] = rd16(in + 20 + 2 * i);
    cmf[0] = 0;
    cmf[1] = pmf[0];
    cmf[2] = cmf[1] + pmf[1];
    uint32_t tot = cmf[2] + pmf[2];
    if (tot == 0) return -1;
    const uint8_t *pay = in + 26;
    size_t nbytes = (size_t)((nbits + 7) / 8), pos = 0;
    if ((int64_t)nbytes > in_size - 26) return -1;
#define NEXTBYTE() (pos < nbytes ? pay[pos++] : (uint8_t)0)
    uint32_t low = 0, range = 0xFFFFFFFFu, sr = 0;
    for (int i = 0; i < 4; i++) sr = (sr << 8) | NEXTBYTE();
    int64_t qcols = (columns + 15) / 16;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t qc = 0; qc < qcols; qc++) {
            uint32_t w = 0;
            int lim = (int)((columns - qc * 16) < 16 ? (columns - qc * 16) : 16);
            for (int i = 0; i < lim; i++) {
                range /= tot;
                if (range == 0) return -1;
                uint32_t freq = (sr - low) / range;
                /* binary search of tmq/rangecoder.h:177-185 */
                int lo = 0, hi = 3, s;
                for (;;) {
                    int mid = (lo + hi) / 2;
                    if (cmf[mid] > freq) hi = mid;
                    else if (mid >= 2 || cmf[mid + 1] > freq) { s = mid; break; }
                    else lo = mid;
                }
                low += cmf[s] * range;
                range *= pmf[s];
                while (renorm_needed(low, &range)) {
                    sr = (sr << 8) | NEXTBYTE();
                    range <<= 8;
                    low <<= 8;
                }
                w = (w << 2) | codetable[s];
            }
            if (lim != 16) w <<= 2 * (16 - lim);
            words[r * qcols + qc] = w;
        }
#undef NEXTBYTE
    return (int64_t)numsyms;
}
