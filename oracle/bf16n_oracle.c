/* TEST INFRASTRUCTURE ONLY — see bf16n_oracle.h.  Plain C99, no dependencies beyond libc/libm (+ OpenMP if enabled). */
#include "bf16n_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define MAGIC 0x4e363142u /* "B16N", core/include/bf16n/format.h:17 */
#define HUF_LMAX 10       /* format.h:18 */
#define HP_LP 12          /* format.h:20 */
#define CHUNK 512         /* format.h:24 */
#define K_MAX 4096        /* format.h:25 */

static _Thread_local char g_err[256];
const char *orc_last_error(void) { return g_err; }
static int fail(const char *msg) {
    snprintf(g_err, sizeof g_err, "bf16n encode: %s", msg);
    return -1;
}
void orc_free(void *p) { free(p); }

int orc_pos_of(int l, int s) { return 128 * (s >> 2) + 4 * l + (s & 3); }

static inline int ex_of(uint16_t v) { return (v >> 7) & 0xFF; }
static inline uint8_t sm_of(uint16_t v) { return (uint8_t) (((v >> 15) << 7) | (v & 0x7F)); }
static inline uint16_t join(uint8_t sm, int ex) { return (uint16_t) (((sm >> 7) << 15) | (ex << 7) | (sm & 0x7F)); }
static inline float bf16_to_f(uint16_t v) {
    uint32_t b = (uint32_t) v << 16;
    float f;
    memcpy(&f, &b, 4);
    return f;
}

/* ---------------------------------------------------------------- plane (encode.cpp:48-62) */
void orc_plane(const uint16_t *w, int64_t rows, int64_t K, uint8_t *plane) {
    const int64_t C = K / CHUNK;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < C; c++)
            for (int l = 0; l < 32; l++)
                for (int s = 0; s < 16; s++)
                    plane[r * K + c * CHUNK + 16 * l + s] = sm_of(w[r * K + c * CHUNK + orc_pos_of(l, s)]);
}

/* ---------------------------------------------------------------- package-merge (encode.cpp:182-218)
 * The reference keeps explicit symbol sets per item; the same selection is computed here by counting: the items chosen at
 * level d are a prefix of that level's list, the packages among them are a prefix of the package list and so select
 * the first 2p items one level down; a leaf gains one bit per level in which it lies inside the chosen prefix. */
typedef struct { uint64_t w; int sym; } leaf_t;
static int leaf_cmp(const void *a, const void *b) {
    const leaf_t *x = a, *y = b;
    if (x->w != y->w) return x->w < y->w ? -1 : 1;
    return x->sym - y->sym;
}
void orc_limited_lengths(const uint64_t *freq, int nfreq, int L, int *len) {
    int n = 0;
    for (int i = 0; i < nfreq; i++) { len[i] = 0; n += freq[i] != 0; }
    if (n == 0) return;
    leaf_t *leaves = malloc((size_t) n * sizeof *leaves);
    for (int i = 0, k = 0; i < nfreq; i++)
        if (freq[i]) { leaves[k].w = freq[i]; leaves[k].sym = i; k++; }
    if (n == 1) { len[leaves[0].sym] = 1; free(leaves); return; }
    qsort(leaves, (size_t) n, sizeof *leaves, leaf_cmp);
    /* level lists: weights and is-package flags; level 1 = leaves, level d = merge(packages(level d-1), leaves) */
    const int cap = 2 * n;
    uint64_t *wt = malloc((size_t) L * cap * sizeof *wt);
    uint8_t *pk = malloc((size_t) L * cap);
    int *cnt = malloc((size_t) L * sizeof *cnt);
    for (int i = 0; i < n; i++) { wt[i] = leaves[i].w; pk[i] = 0; }
    cnt[0] = n;
    for (int d = 1; d < L; d++) {
        const uint64_t *pw = wt + (size_t) (d - 1) * cap;
        uint64_t *cw = wt + (size_t) d * cap;
        uint8_t *cp = pk + (size_t) d * cap;
        const int np = cnt[d - 1] / 2;
        int i = 0, j = 0, k = 0;
        while (i < np || j < n) {
            /* std::merge(pk, leaves): a leaf goes first only when strictly lighter than the package */
            if (i < np && (j >= n || !(leaves[j].w < pw[2 * i] + pw[2 * i + 1]))) {
                cw[k] = pw[2 * i] + pw[2 * i + 1]; cp[k] = 1; i++;
            } else {
                cw[k] = leaves[j].w; cp[k] = 0; j++;
            }
            k++;
        }
        cnt[d] = k;
    }
    int m = 2 * n - 2;
    for (int d = L - 1; d >= 0; d--) {
        if (m > cnt[d]) m = cnt[d]; /* cannot happen when n <= 2^L */
        const uint8_t *cp = pk + (size_t) d * cap;
        int p = 0;
        for (int i = 0; i < m; i++) p += cp[i];
        const int q = m - p;
        for (int i = 0; i < q; i++) len[leaves[i].sym]++;
        m = 2 * p;
    }
    free(cnt); free(pk); free(wt); free(leaves);
}

/* canonical codes from lengths (encode.cpp:239-250, :348-358) */
static void canonical(const int *len, int n, int L, uint32_t *code) {
    uint32_t c = 0;
    for (int l = 1; l <= L; l++) {
        for (int s = 0; s < n; s++)
            if (len[s] == l) code[s] = c++;
        c <<= 1;
    }
}

/* ---------------------------------------------------------------- growable word buffer + MSB-first bit writer */
typedef struct { uint32_t *p; size_t n, cap; } wbuf;
static void wb_push(wbuf *b, uint32_t v) {
    if (b->n == b->cap) { b->cap = b->cap ? 2 * b->cap : 256; b->p = realloc(b->p, b->cap * 4); }
    b->p[b->n++] = v;
}
typedef struct { wbuf *out; uint64_t acc; int nb; } bitw;
static void bw_put(bitw *b, uint32_t code, int len) { /* encode.cpp:377-386 */
    b->acc = (b->acc << len) | code;
    b->nb += len;
    if (b->nb >= 32) {
        wb_push(b->out, (uint32_t) (b->acc >> (b->nb - 32)));
        b->nb -= 32;
        b->acc &= b->nb ? ((1ull << b->nb) - 1) : 0;
    }
}
static void bw_flush(bitw *b) { /* encode.cpp:404-406 */
    if (b->nb) wb_push(b->out, (uint32_t) (b->acc << (32 - b->nb)));
    b->acc = 0; b->nb = 0;
}

/* ---------------------------------------------------------------- NIBBLE (encode.cpp:94-180, :482-493) */
static uint8_t *encode_nibble(const uint16_t *w, int64_t rows, int64_t K, uint8_t *plane, uint64_t *aux_bytes) {
    const int64_t C = K / CHUNK;
    uint8_t *nib = calloc((size_t) (rows * K / 2), 1);
    uint8_t *lut = calloc((size_t) rows * 16, 1);
    uint32_t *esc_off = calloc((size_t) rows + 1, 4);
    wbuf esc = {0};
    for (int64_t r = 0; r < rows; r++) {
        const uint16_t *row = w + r * K;
        int hist[256] = {0}, idx[256], code_of[256];
        for (int64_t k = 0; k < K; k++) hist[ex_of(row[k])]++;
        for (int i = 0; i < 256; i++) { idx[i] = i; code_of[i] = -1; }
        /* order: count descending, ties by smaller exponent (encode.cpp:113) — a total order, so any sort agrees */
        for (int i = 1; i < 256; i++) {
            const int v = idx[i];
            int j = i - 1;
            while (j >= 0 && (hist[idx[j]] < hist[v] || (hist[idx[j]] == hist[v] && idx[j] > v))) { idx[j + 1] = idx[j]; j--; }
            idx[j + 1] = v;
        }
        code_of[0] = 0;
        int n = 1;
        for (int i = 0; i < 256 && n < 16; i++) {
            const int x = idx[i];
            if (hist[x] == 0) break;
            if (x == 0 || x >= 128) continue;
            lut[r * 16 + n] = (uint8_t) x;
            code_of[x] = n++;
        }
        for (int64_t c = 0; c < C; c++) {
            for (int l = 0; l < 32; l++) {
                uint32_t nw[2] = {0, 0};
                for (int s = 0; s < 16; s++) {
                    const int col = (int) (c * CHUNK + orc_pos_of(l, s));
                    const uint16_t v = row[col];
                    int code = code_of[ex_of(v)];
                    if (code < 0) {
                        wb_push(&esc, (uint32_t) col | ((uint32_t) sm_of(v) << 12) | ((uint32_t) ex_of(v) << 20));
                        plane[r * K + c * CHUNK + 16 * l + s] = 0; /* escaped weights read as +0 in the plane */
                        code = 0;
                    }
                    nw[s >> 3] |= (uint32_t) code << (4 * (s & 7));
                }
                memcpy(nib + (r * C + c) * 256 + 8 * l, nw, 8);
            }
        }
        esc_off[r + 1] = (uint32_t) esc.n;
    }
    orc_header h;
    memset(&h, 0, sizeof h);
    h.magic = MAGIC; h.format = ORC_FMT_NIBBLE; h.K = (uint32_t) K; h.rows = (uint64_t) rows;
    h.off_a = 256;
    h.off_b = h.off_a + (uint64_t) (rows * K / 2);
    h.off_c = h.off_b + (uint64_t) rows * 16;
    h.off_d = h.off_c + ((uint64_t) rows + 1) * 4;
    h.n_a = esc.n;
    const uint64_t total = h.off_d + (esc.n ? esc.n : 1) * 4;
    uint8_t *aux = calloc(total, 1);
    memcpy(aux, &h, sizeof h);
    memcpy(aux + h.off_a, nib, (size_t) (rows * K / 2));
    memcpy(aux + h.off_b, lut, (size_t) rows * 16);
    memcpy(aux + h.off_c, esc_off, ((size_t) rows + 1) * 4);
    if (esc.n) memcpy(aux + h.off_d, esc.p, esc.n * 4);
    free(nib); free(lut); free(esc_off); free(esc.p);
    *aux_bytes = total;
    return aux;
}

/* ---------------------------------------------------------------- HUFFMAN single symbol (encode.cpp:220-312) */
static uint8_t *encode_huffman(const uint16_t *w, int64_t rows, int64_t K, int R, uint64_t *aux_bytes) {
    const int64_t C = K / CHUNK, units = rows / R;
    uint64_t freq[256] = {0};
    for (int64_t i = 0; i < rows * K; i++) freq[ex_of(w[i])]++;
    int len[256];
    uint32_t code[256] = {0};
    orc_limited_lengths(freq, 256, HUF_LMAX, len);
    canonical(len, 256, HUF_LMAX, code);
    uint32_t *lut = calloc(1 << HUF_LMAX, 4);
    for (int s = 0; s < 256; s++)
        if (len[s])
            for (uint32_t i = code[s] << (HUF_LMAX - len[s]); i < (code[s] + 1) << (HUF_LMAX - len[s]); i++)
                lut[i] = (uint32_t) len[s] | ((uint32_t) s << 7);
    wbuf st = {0};
    uint32_t *lane_off = malloc((size_t) units * 32 * 4);
    for (int64_t u = 0; u < units; u++)
        for (int l = 0; l < 32; l++) {
            lane_off[u * 32 + l] = (uint32_t) st.n;
            bitw b = {&st, 0, 0};
            for (int64_t r = u * R; r < (u + 1) * R; r++)
                for (int64_t c = 0; c < C; c++)
                    for (int s = 0; s < 16; s++) {
                        const int e = ex_of(w[r * K + c * CHUNK + orc_pos_of(l, s)]);
                        bw_put(&b, code[e], len[e]);
                    }
            bw_flush(&b);
        }
    orc_header h;
    memset(&h, 0, sizeof h);
    h.magic = MAGIC; h.format = ORC_FMT_HUFFMAN; h.K = (uint32_t) K; h.R = (uint32_t) R; h.rows = (uint64_t) rows;
    h.off_a = 256;
    h.off_b = h.off_a + (4u << HUF_LMAX);
    h.off_c = h.off_b + (uint64_t) units * 32 * 4;
    h.n_a = (uint64_t) units; h.n_b = st.n;
    const uint64_t total = h.off_c + (st.n + 16) * 4; /* +16 words of decoder lookahead (encode.cpp:302) */
    uint8_t *aux = calloc(total, 1);
    memcpy(aux, &h, sizeof h);
    memcpy(aux + h.off_a, lut, 4u << HUF_LMAX);
    memcpy(aux + h.off_b, lane_off, (size_t) units * 32 * 4);
    if (st.n) memcpy(aux + h.off_c, st.p, st.n * 4);
    free(lut); free(lane_off); free(st.p);
    *aux_bytes = total;
    return aux;
}

/* ---------------------------------------------------------------- HUFPAIR (encode.cpp:321-439); NULL = too many pairs */
static uint8_t *encode_hufpair(const uint16_t *w, int64_t rows, int64_t K, int R, int cm, uint64_t *aux_bytes) {
    const int64_t C = K / CHUNK, units = rows / R;
    uint64_t *freq = calloc(65536, 8);
    for (int64_t i = 0; i < rows * K; i += 2) freq[ex_of(w[i]) | ex_of(w[i + 1]) << 8]++;
    int nsym = 0;
    for (int i = 0; i < 65536; i++) nsym += freq[i] != 0;
    if (nsym > (1 << HP_LP)) { free(freq); return NULL; }
    int *len = malloc(65536 * sizeof *len);
    uint32_t *code = calloc(65536, 4);
    orc_limited_lengths(freq, 65536, HP_LP, len);
    canonical(len, 65536, HP_LP, code);
    uint32_t *lut = calloc(1 << HP_LP, 4);
    for (int s = 0; s < 65536; s++)
        if (len[s])
            for (uint32_t i = code[s] << (HP_LP - len[s]); i < (code[s] + 1) << (HP_LP - len[s]); i++)
                lut[i] = ((uint32_t) (s >> 8) << 23) | ((uint32_t) (s & 0xFF) << 7) | (uint32_t) len[s];
    wbuf st = {0};
    uint32_t *unit_base = malloc((size_t) units * 4);
    uint16_t *lane_rel = malloc((size_t) units * 32 * 2);
    int bad = 0;
    for (int64_t u = 0; u < units; u++) {
        unit_base[u] = (uint32_t) st.n;
        for (int l = 0; l < 32; l++) {
            const size_t rel = st.n - unit_base[u];
            if (rel > 0xFFFF) bad = 1; /* encode.cpp:415 */
            lane_rel[u * 32 + l] = (uint16_t) rel;
            bitw b = {&st, 0, 0};
            for (int64_t o = 0; o < R * C; o++) {
                const int64_t r = u * R + (cm ? o % R : o / C), c = cm ? o / R : o % C;
                for (int s = 0; s < 16; s += 2) {
                    const int64_t i = r * K + c * CHUNK + orc_pos_of(l, s);
                    const int sym = ex_of(w[i]) | ex_of(w[i + 1]) << 8;
                    bw_put(&b, code[sym], len[sym]);
                }
            }
            bw_flush(&b);
        }
    }
    uint8_t *aux = NULL;
    if (!bad && st.n + 32 < (1ull << 32)) {
        orc_header h;
        memset(&h, 0, sizeof h);
        h.magic = MAGIC; h.format = ORC_FMT_HUFPAIR; h.K = (uint32_t) K; h.R = (uint32_t) R; h.rows = (uint64_t) rows;
        h.off_a = 256;
        h.off_b = h.off_a + (4u << HP_LP);
        h.off_c = h.off_b + (uint64_t) units * 4;
        h.off_d = (h.off_c + (uint64_t) units * 32 * 2 + 15) & ~15ull;
        h.n_a = (uint64_t) units; h.n_b = st.n; h.flags = cm ? ORC_FLAG_CHUNK_MAJOR : 0;
        const uint64_t total = h.off_d + (st.n + 32) * 4; /* +32 words of lookahead (encode.cpp:428) */
        aux = calloc(total, 1);
        memcpy(aux, &h, sizeof h);
        memcpy(aux + h.off_a, lut, 4u << HP_LP);
        memcpy(aux + h.off_b, unit_base, (size_t) units * 4);
        memcpy(aux + h.off_c, lane_rel, (size_t) units * 32 * 2);
        if (st.n) memcpy(aux + h.off_d, st.p, st.n * 4);
        *aux_bytes = total;
    } else {
        snprintf(g_err, sizeof g_err, "bf16n encode: check failed: lane offset / stream size");
    }
    free(freq); free(len); free(code); free(lut); free(unit_base); free(lane_rel); free(st.p);
    return aux;
}

/* ---------------------------------------------------------------- encode() (encode.cpp:443-526) */
int orc_encode(const uint16_t *w, int64_t rows, int64_t K, int format, int R, int cm, uint8_t *plane, uint8_t **aux,
               uint64_t *aux_bytes, int *format_out) {
    if (K % CHUNK != 0 || K < CHUNK || K > K_MAX) return fail("K must be a multiple of 512 in [512, 4096]");
    if (rows <= 0) return fail("rows must be positive");
    if (format == ORC_FMT_NIBBLE) {
        if (R != 0 || cm) return fail("NIBBLE takes R = 0 and no chunk-major or fragment-order layout");
    } else if (format == ORC_FMT_HUFFMAN || format == ORC_FMT_HUFPAIR) {
        if (R != 1 && R != 2 && R != 4 && R != 8 && R != 16) return fail("R must be one of 1, 2, 4, 8, 16");
        if (rows % R != 0) return fail("rows must be a multiple of R");
        if (format == ORC_FMT_HUFFMAN && cm) return fail("chunk-major units exist only for HUFPAIR");
        if (cm && (K == CHUNK || (R != 4 && R != 8 && R != 16))) return fail("chunk-major units need K > 512 and R in {4, 8, 16}");
    } else {
        return fail("unknown format");
    }
    orc_plane(w, rows, K, plane);
    if (format == ORC_FMT_NIBBLE) {
        *aux = encode_nibble(w, rows, K, plane, aux_bytes);
        *format_out = ORC_FMT_NIBBLE;
        return 0;
    }
    *aux = NULL;
    if (format == ORC_FMT_HUFPAIR) *aux = encode_hufpair(w, rows, K, R, cm, aux_bytes);
    if (*aux) {
        *format_out = ORC_FMT_HUFPAIR;
    } else {
        *aux = encode_huffman(w, rows, K, R, aux_bytes);
        *format_out = ORC_FMT_HUFFMAN;
        cm = 0;
    }
    if (cm) { /* chunk-major plane: chunk c of unit row r at (c*R + r)*512 inside the unit (encode.cpp:511-524) */
        uint8_t *tmp = malloc((size_t) (R * K));
        for (int64_t u = 0; u < rows / R; u++) {
            uint8_t *ub = plane + u * R * K;
            memcpy(tmp, ub, (size_t) (R * K));
            for (int r = 0; r < R; r++)
                for (int64_t c = 0; c < K / CHUNK; c++) memcpy(ub + (c * R + r) * CHUNK, tmp + r * K + c * CHUNK, CHUNK);
        }
        free(tmp);
    }
    return 0;
}

/* ---------------------------------------------------------------- independent decoder (test_encode.cpp:36-164) */
typedef struct { const uint8_t *b; uint64_t base, word; uint64_t acc; int n; } bitr;
static uint32_t rd32(const uint8_t *b, uint64_t off) { uint32_t v; memcpy(&v, b + off, 4); return v; }
static uint32_t br_peek(bitr *r, int k) {
    while (r->n < k) { r->acc = (r->acc << 32) | rd32(r->b, r->base + 4 * r->word++); r->n += 32; }
    return (uint32_t) ((r->acc >> (r->n - k)) & ((1ull << k) - 1));
}
static void br_skip(bitr *r, int k) { r->n -= k; r->acc &= r->n ? ((1ull << r->n) - 1) : 0; }

/* plane byte of weight (r, col); chunk-major units keep chunk c of unit row r at (c*R + r%R)*512 */
static uint8_t sm_at(const uint8_t *plane, int64_t K, int64_t R, int64_t r, int64_t col, int cm) {
    const int64_t c = col / CHUNK, p = col % CHUNK;
    const int64_t in_chunk = 16 * ((p % 128) / 4) + 4 * (p / 128) + p % 4; /* inverse of pos_of */
    if (cm) return plane[(r / R) * R * K + (c * R + r % R) * CHUNK + in_chunk];
    return plane[r * K + c * CHUNK + in_chunk];
}

static int decode_exponents(const uint8_t *aux, uint64_t aux_bytes, const orc_header *h, int *ex) {
    const int64_t K = h->K, rows = (int64_t) h->rows, C = K / CHUNK;
    const int cm = (h->flags & ORC_FLAG_CHUNK_MAJOR) != 0;
    (void) aux_bytes;
    if (h->format == ORC_FMT_NIBBLE) {
        for (int64_t r = 0; r < rows; r++)
            for (int64_t c = 0; c < C; c++)
                for (int l = 0; l < 32; l++) {
                    uint64_t nw;
                    memcpy(&nw, aux + h->off_a + (r * C + c) * 256 + 8 * l, 8);
                    for (int s = 0; s < 16; s++)
                        ex[r * K + c * CHUNK + orc_pos_of(l, s)] = aux[h->off_b + r * 16 + ((nw >> (4 * s)) & 0xF)];
                }
    } else if (h->format == ORC_FMT_HUFFMAN) {
        for (uint64_t u = 0; u < h->n_a; u++)
            for (int l = 0; l < 32; l++) {
                bitr bs = {aux, h->off_c, rd32(aux, h->off_b + 4 * (u * 32 + l)), 0, 0};
                for (int64_t r = (int64_t) u * h->R; r < (int64_t) (u + 1) * h->R; r++)
                    for (int64_t c = 0; c < C; c++)
                        for (int s = 0; s < 16; s++) {
                            const uint32_t v = rd32(aux, h->off_a + 4 * br_peek(&bs, HUF_LMAX));
                            br_skip(&bs, (int) (v & 0x7F));
                            ex[r * K + c * CHUNK + orc_pos_of(l, s)] = (int) ((v >> 7) & 0xFF);
                        }
            }
    } else if (h->format == ORC_FMT_HUFPAIR) {
        for (uint64_t u = 0; u < h->n_a; u++) {
            const uint32_t ub = rd32(aux, h->off_b + 4 * u);
            for (int l = 0; l < 32; l++) {
                uint16_t rel;
                memcpy(&rel, aux + h->off_c + 2 * (u * 32 + l), 2);
                bitr bs = {aux, h->off_d, (uint64_t) ub + rel, 0, 0};
                for (int64_t o = 0; o < (int64_t) h->R * C; o++) {
                    const int64_t r = (int64_t) u * h->R + (cm ? o % h->R : o / C), c = cm ? o / h->R : o % C;
                    for (int s = 0; s < 16; s += 2) {
                        const uint32_t v = rd32(aux, h->off_a + 4 * br_peek(&bs, HP_LP));
                        br_skip(&bs, (int) (v & 0x7F));
                        ex[r * K + c * CHUNK + orc_pos_of(l, s)] = (int) ((v >> 7) & 0xFF);
                        ex[r * K + c * CHUNK + orc_pos_of(l, s + 1)] = (int) ((v >> 23) & 0xFF);
                    }
                }
            }
        }
    } else {
        return -1;
    }
    return 0;
}

int orc_decode(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, uint16_t *out) {
    orc_header h;
    if (aux_bytes < 256) return -1;
    memcpy(&h, aux, sizeof h);
    if (h.magic != MAGIC || h.K % CHUNK || h.K < CHUNK || h.K > K_MAX) return -1;
    if (h.flags & ORC_FLAG_WAVE64) return orc_decode_w64(plane, aux, aux_bytes, out);
    const int64_t K = h.K, rows = (int64_t) h.rows;
    const int cm = (h.flags & ORC_FLAG_CHUNK_MAJOR) != 0;
    int *ex = malloc((size_t) (rows * K) * sizeof *ex);
    if (decode_exponents(aux, aux_bytes, &h, ex)) { free(ex); return -1; }
    for (int64_t r = 0; r < rows; r++)
        for (int64_t k = 0; k < K; k++) out[r * K + k] = join(sm_at(plane, K, h.R ? h.R : 1, r, k, cm), ex[r * K + k]);
    if (h.format == ORC_FMT_NIBBLE) /* escapes: column | sign|mantissa << 12 | exponent << 20 */
        for (int64_t r = 0; r < rows; r++)
            for (uint32_t i = rd32(aux, h.off_c + 4 * r); i < rd32(aux, h.off_c + 4 * (r + 1)); i++) {
                const uint32_t x = rd32(aux, h.off_d + 4 * i);
                out[r * K + (x & 0xFFF)] = join((uint8_t) ((x >> 12) & 0xFF), (int) (x >> 20));
            }
    free(ex);
    return 0;
}

/* ---------------------------------------------------------------- wave64 layout decoder
 * HUFPAIR with flag bit 2.  A unit is R rows decoded by 64 lanes.  The unit's 512-column chunks are taken in stream order
 * o = 0 .. R*C-1 (row-major o -> (o / C, o % C), chunk-major o -> (o % R, o / R)); lanes 0..31 own chunk 2i, lanes
 * 32..63 chunk 2i+1 of step i, each with the reference (lane, slot) ownership, so the plane is the reference plane.
 * Every lane has a bit sequence: 2 zero bits, then its pair codes, each code written first-bit-lowest; 32-bit word k of
 * the lane holds sequence bits [32k, 32k+32) with bit j of the word = sequence bit 32k+j.  The LUT at off_a is indexed
 * by the next 12 sequence bits (first bit = index bit 0).  A lane holds three words (w0, w1, w2) and a position P into
 * w0; after every second pair it adds the two code lengths to P and, if P >= 32, takes the unit stream's next word
 * (lanes in ascending order) as its new w2, moves w2 to w1 and w1 to w0 and subtracts 32.  The unit stream is: the
 * lanes' first three words (lane 0 words 0, 1, 2, lane 1 words 0, 1, 2, ...), then the refill words in the order taken.
 * off_b: u32 unit_base[units + 1] (word index of each unit's stream), off_d: words. */
static int decode_w64_units(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, orc_header h, uint16_t *out) {
    const int64_t K = h.K, C = K / CHUNK, R = h.R;
    const int cm = (h.flags & ORC_FLAG_CHUNK_MAJOR) != 0;
    if ((R * C) % 2) return -1;
    for (uint64_t u = 0; u < h.n_a; u++) {
        uint64_t next = h.off_d + 4ull * rd32(aux, h.off_b + 4 * u);
        uint32_t w0[64], w1[64], w2[64], P[64];
        for (int l = 0; l < 64; l++) {
            w0[l] = rd32(aux, next); w1[l] = rd32(aux, next + 4); w2[l] = rd32(aux, next + 8);
            next += 12; P[l] = 0;
        }
        for (int64_t step = 0; step < R * C / 2; step++) {
            for (int q = 0; q < 8; q += 2) {
                for (int l = 0; l < 64; l++) {
                    const int64_t o = 2 * step + (l >> 5);
                    const int64_t r = (int64_t) u * R + (cm ? o % R : o / C), c = cm ? o / R : o % C;
                    const uint64_t win = (((uint64_t) w1[l] << 32) | w0[l]) >> P[l];
                    uint32_t used = 0;
                    for (int k = 0; k < 2; k++) {
                        const uint32_t idx = (uint32_t) (win >> (2 + used)) & 0xFFF;
                        const uint32_t v = rd32(aux, h.off_a + 4 * idx);
                        used += v & 0x7F;
                        const int s = 2 * (q + k);
                        const int64_t col = c * CHUNK + orc_pos_of(l & 31, s);
                        out[r * K + col] = join(sm_at(plane, K, R, r, col, cm), (int) ((v >> 7) & 0xFF));
                        out[r * K + col + 1] = join(sm_at(plane, K, R, r, col + 1, cm), (int) ((v >> 23) & 0xFF));
                    }
                    P[l] += used;
                }
                for (int l = 0; l < 64; l++)
                    if (P[l] >= 32) {
                        if (next + 4 > aux_bytes) return -1;
                        w0[l] = w1[l]; w1[l] = w2[l]; w2[l] = rd32(aux, next); next += 4; P[l] -= 32;
                    }
            }
        }
        if (next != h.off_d + 4ull * rd32(aux, h.off_b + 4 * (u + 1))) return -1; /* stream length must match exactly */
    }
    return 0;
}

/* R = 32 (only with flag bit 2): tiles in matrix-core operand order.  Unit u = g * (K / 256) + t holds rows
 * [32 g, 32 g + 32) x columns [256 t, 256 t + 256); it is stored exactly as a wave64 unit of 16 rows of a 512-column
 * matrix V (plane and stream), where V[16 u + 2 s + h][128 j + 4 l + q] = W[32 g + l][256 t + 32 s + 16 (j / 2) + 8 h
 * + 4 (j % 2) + q] for s < 8, h < 2, j < 4, l < 32, q < 4: in step s lane 32 h + l holds, in slot order, columns
 * 32 s + 8 h + [0, 8) and 32 s + 16 + 8 h + [0, 8) of row l of the tile. */
int64_t orc_tile32_index(int64_t vrow, int64_t vcol, int64_t K) {
    const int64_t u = vrow / 16, sh = vrow % 16, s = sh / 2, hh = sh % 2;
    const int64_t j = vcol / 128, l = (vcol % 128) / 4, q = vcol % 4;
    const int64_t slabs = K / 256, g = u / slabs, t = u % slabs;
    return (32 * g + l) * K + 256 * t + 32 * s + 16 * (j / 2) + 8 * hh + 4 * (j % 2) + q;
}

int orc_decode_w64(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, uint16_t *out) {
    orc_header h;
    if (aux_bytes < 256) return -1;
    memcpy(&h, aux, sizeof h);
    if (h.magic != MAGIC || h.format != ORC_FMT_HUFPAIR || !(h.flags & ORC_FLAG_WAVE64) || h.R == 0) return -1;
    if (h.R != 32) return decode_w64_units(plane, aux, aux_bytes, h, out);
    if ((h.flags & ORC_FLAG_CHUNK_MAJOR) || h.rows % 32 || h.K % 256) return -1;
    const int64_t K = h.K, n = (int64_t) h.rows * K, vrows = n / CHUNK;
    orc_header v = h;
    v.K = CHUNK; v.R = 16; v.rows = (uint64_t) vrows;
    uint16_t *tmp = (uint16_t *) malloc((size_t) n * 2);
    if (!tmp) return -1;
    int rc = decode_w64_units(plane, aux, aux_bytes, v, tmp);
    if (rc == 0)
        for (int64_t r = 0; r < vrows; r++)
            for (int64_t c = 0; c < CHUNK; c++) out[orc_tile32_index(r, c, K)] = tmp[r * CHUNK + c];
    free(tmp);
    return rc;
}

/* ---------------------------------------------------------------- GEMV references */
static float lane_tree32(float *v) { /* kernels.cuh:119-125: v += shfl_xor(v, o), o = 16..1, every lane at once */
    for (int o = 16; o; o >>= 1) {
        float t[32];
        for (int l = 0; l < 32; l++) t[l] = v[l] + v[l ^ o];
        memcpy(v, t, sizeof t);
    }
    return v[0];
}

/* dot of one row held as BF16 bits in the lane order of the kernels; esc (optional): records of this row */
static float row_dot_f32(const uint16_t *row, int64_t K, const float *x, int cm, const uint32_t *esc, uint32_t n_esc) {
    const int64_t C = K / CHUNK;
    float lane[32];
    for (int l = 0; l < 32; l++) {
        float acc = 0.f, a[4] = {0.f, 0.f, 0.f, 0.f};
        for (int64_t c = 0; c < C; c++) {
            if (cm) a[0] = a[1] = a[2] = a[3] = 0.f;
            for (int j = 0; j < 4; j++)
                for (int t = 0; t < 4; t++) {
                    const int64_t col = c * CHUNK + 128 * j + 4 * l + t;
                    a[t] = fmaf(bf16_to_f(row[col]), x[col], a[t]);
                }
            if (cm) acc += (a[0] + a[1]) + (a[2] + a[3]); /* kernels.cuh:969 */
        }
        if (!cm) acc = (a[0] + a[1]) + (a[2] + a[3]); /* kernels.cuh:534 */
        for (uint32_t i = (uint32_t) l; i < n_esc; i += 32) { /* kernels.cuh:179-185 */
            const uint32_t rec = esc[i];
            acc = fmaf(bf16_to_f(join((uint8_t) ((rec >> 12) & 0xFF), (int) (rec >> 20))), x[rec & 0xFFF], acc);
        }
        lane[l] = acc;
    }
    return lane_tree32(lane);
}

void orc_gemv_f32(const uint16_t *w, int64_t rows, int64_t K, const float *x, int cm, float *y) {
    for (int64_t r = 0; r < rows; r++) y[r] = row_dot_f32(w + r * K, K, x, cm, NULL, 0);
}

void orc_gemv_f64(const uint16_t *w, int64_t rows, int64_t K, const float *x, double *y, double *s) {
    for (int64_t r = 0; r < rows; r++) {
        double a = 0, b = 0;
        for (int64_t k = 0; k < K; k++) {
            const double p = (double) bf16_to_f(w[r * K + k]) * (double) x[k];
            a += p; b += fabs(p);
        }
        y[r] = a;
        if (s) s[r] = b;
    }
}

/* decode one unit (reference layouts) or one NIBBLE row into BF16 bits; used by orc_decode_gemv */
static void decode_unit_rows(const uint8_t *plane, const uint8_t *aux, const orc_header *h, int64_t u, uint16_t *rows_out) {
    const int64_t K = h->K, C = K / CHUNK, R = h->R;
    const int cm = (h->flags & ORC_FLAG_CHUNK_MAJOR) != 0;
    for (int l = 0; l < 32; l++) {
        bitr bs;
        if (h->format == ORC_FMT_HUFPAIR) {
            uint16_t rel;
            memcpy(&rel, aux + h->off_c + 2 * (u * 32 + l), 2);
            bs = (bitr){aux, h->off_d, (uint64_t) rd32(aux, h->off_b + 4 * u) + rel, 0, 0};
        } else {
            bs = (bitr){aux, h->off_c, rd32(aux, h->off_b + 4 * (u * 32 + l)), 0, 0};
        }
        for (int64_t o = 0; o < R * C; o++) {
            const int64_t rr = cm ? o % R : o / C, c = cm ? o / R : o % C;
            const uint8_t *pl = plane + u * R * K + (cm ? (c * R + rr) * CHUNK : rr * K + c * CHUNK) + 16 * l;
            uint16_t *dst = rows_out + rr * K + c * CHUNK;
            if (h->format == ORC_FMT_HUFPAIR) {
                for (int s = 0; s < 16; s += 2) {
                    const uint32_t v = rd32(aux, h->off_a + 4 * br_peek(&bs, HP_LP));
                    br_skip(&bs, (int) (v & 0x7F));
                    dst[orc_pos_of(l, s)] = join(pl[s], (int) ((v >> 7) & 0xFF));
                    dst[orc_pos_of(l, s + 1)] = join(pl[s + 1], (int) ((v >> 23) & 0xFF));
                }
            } else {
                for (int s = 0; s < 16; s++) {
                    const uint32_t v = rd32(aux, h->off_a + 4 * br_peek(&bs, HUF_LMAX));
                    br_skip(&bs, (int) (v & 0x7F));
                    dst[orc_pos_of(l, s)] = join(pl[s], (int) ((v >> 7) & 0xFF));
                }
            }
        }
    }
}

int orc_decode_gemv(const uint8_t *plane, const uint8_t *aux, uint64_t aux_bytes, int64_t row0, int64_t nrows,
                    const float *x, float *y, int threads) {
    orc_header h;
    if (aux_bytes < 256) return -1;
    memcpy(&h, aux, sizeof h);
    if (h.magic != MAGIC || (h.flags & ORC_FLAG_WAVE64)) return -1;
    const int64_t K = h.K, C = K / CHUNK;
    const int cm = (h.flags & ORC_FLAG_CHUNK_MAJOR) != 0;
    (void) threads;
    if (h.format == ORC_FMT_NIBBLE) {
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
#endif
        for (int64_t r = row0; r < row0 + nrows; r++) {
            uint16_t row[K_MAX];
            for (int64_t c = 0; c < C; c++)
                for (int l = 0; l < 32; l++) {
                    uint64_t nw;
                    memcpy(&nw, aux + h.off_a + (r * C + c) * 256 + 8 * l, 8);
                    for (int s = 0; s < 16; s++)
                        row[c * CHUNK + orc_pos_of(l, s)] =
                            join(plane[r * K + c * CHUNK + 16 * l + s], aux[h.off_b + r * 16 + ((nw >> (4 * s)) & 0xF)]);
                }
            const uint32_t e0 = rd32(aux, h.off_c + 4 * r), e1 = rd32(aux, h.off_c + 4 * (r + 1));
            y[r - row0] = row_dot_f32(row, K, x, 0, (const uint32_t *) (aux + h.off_d) + e0, e1 - e0);
        }
        return 0;
    }
    const int64_t R = h.R;
    if (row0 % R || nrows % R) return -1;
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
#endif
    for (int64_t u = row0 / R; u < (row0 + nrows) / R; u++) {
        uint16_t *buf = malloc((size_t) (R * K) * 2);
        decode_unit_rows(plane, aux, &h, u, buf);
        for (int64_t rr = 0; rr < R; rr++) y[u * R + rr - row0] = row_dot_f32(buf + rr * K, K, x, cm, NULL, 0);
        free(buf);
    }
    return 0;
}

/* ---------------------------------------------------------------- MoE glue */
void orc_swiglu(const float *g, const float *u, float *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = g[i] / (1.0f + expf(-g[i])) * u[i];
}

void orc_moe_combine(const float *ys, const float *w, float *y, int n_tok, int n_used, int64_t n) {
    for (int t = 0; t < n_tok; t++)
        for (int64_t i = 0; i < n; i++) {
            float acc = 0.f;
            for (int k = 0; k < n_used; k++) {
                const int64_t s = (int64_t) t * n_used + k;
                acc = fmaf(w[s], ys[s * n + i], acc);
            }
            y[(int64_t) t * n + i] = acc;
        }
}

void orc_route(const int32_t *ids, int64_t ids_stride, int n_experts, int n_tok, int n_used, int nchannels_y, int sis1,
               int32_t *ids_src1, int32_t *ids_dst, int32_t *bounds) {
    int listed = 0;
    for (int e = 0; e < n_experts; e++) {
        int j = 0; /* the expert's list starts behind every naming of a lower expert (nex_prev, mmid_helper.cu:66-68) */
        for (int t = 0; t < n_tok; t++)
            for (int k = 0; k < n_used; k++) j += ids[t * ids_stride + k] < e;
        bounds[e] = j;
        for (int t = 0; t < n_tok; t++) {
            int used = -1; /* the last slot of the token naming e (mmid_helper.cu:69-71) */
            for (int k = 0; k < n_used; k++)
                if (ids[t * ids_stride + k] == e) used = k;
            if (used >= 0) {
                ids_dst[j] = t * n_used + used;
                ids_src1[j] = t * sis1 + used % nchannels_y;
                j++;
            }
        }
        listed = j;
    }
    bounds[n_experts] = listed; /* mmid_helper.cu:134 */
}

void orc_router_topk(const float *logits, int n, int k, int32_t *ids, float *weights) {
    float mx = logits[0];
    for (int i = 1; i < n; i++) mx = logits[i] > mx ? logits[i] : mx;
    float *p = malloc((size_t) n * sizeof *p);
    float sum = 0.f;
    for (int i = 0; i < n; i++) { p[i] = expf(logits[i] - mx); sum += p[i]; }
    float top = 0.f;
    for (int j = 0; j < k; j++) {
        int best = -1;
        for (int i = 0; i < n; i++) {
            int taken = 0;
            for (int q = 0; q < j; q++) taken |= ids[q] == i;
            if (!taken && (best < 0 || p[i] > p[best])) best = i;
        }
        ids[j] = best;
        weights[j] = p[best] / sum;
        top += weights[j];
    }
    for (int j = 0; j < k; j++) weights[j] /= top;
    free(p);
}
