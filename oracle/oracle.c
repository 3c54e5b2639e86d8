/*
 * CPU oracle for the condensed-tile SpMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the host-side algorithms and the intended
 * arithmetic of the reference SpMM path so that the HIP implementation can be
 * checked against it.  It is linked only by the test-suite, by the smoke check
 * and by the `cpu_baseline` leg of the benchmark; the product library never
 * links, loads or calls anything in this directory.
 *
 * Each function cites the reference lines it follows (paths relative to the
 * reference checkout).
 *
 * Parity status of each function (what pins it):
 *   orc_f32_to_f16 / orc_f16_to_f32  exhaustive comparison with numpy float16
 *   orc_f32_to_bf16 / orc_bf16_to_f32 comparison with torch.bfloat16 (CPU), all 65536 patterns back
 *   orc_mtx_read                     golden vectors (tiny.mtx, gap.mtx: definition cases small
 *                                    enough to re-derive by hand from the reference's source
 *                                    text), scipy COO->CSR cross-check
 *   orc_btcf_count / orc_btcf_fill   the same golden vectors, round-trip to CSR,
 *                                    brute force on small dense matrices
 *   orc_bitmap_fill                  golden nnzOffset / packed data / as-written tcBit
 *                                    words of tiny.mtx, popcounts, expansion through
 *                                    the set bits equals the uncompressed tiles
 *   orc_group                        hand-computed cases, closed-form group sizes,
 *                                    coverage of every window by its groups
 *   orc_spmm_csr_* / orc_spmm_btcf_* dense numpy float64 product on the same
 *                                    rounded inputs, closed forms, CSR-order vs
 *                                    tile-order agreement
 *   orc_tile_mma_* / orc_tile_accum  closed forms of the reference's micro-tests
 *                                    (256*i+136 and the 1+0.01*i pattern)
 *   orc_verdict_*                    hand-computed cases
 * The reference holds no end-to-end SpMM fixture (its kernel is unfinished), so
 * SpMM-level parity is pinned by the mathematics above, not by reference output.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_IDX_MAX 0xFFFFFFFFu   /* src/common.h:47  IDX_MAX = UINT32_MAX */
#define ORC_ROW_WINDOW 8u         /* src/common.h:17,23,33,40  ROW_WINDOW = 8 */

/* ------------------------------------------------------------------------- */
/* half <-> float, bit level (round to nearest even), as __float2half /      */
/* __half2float do on the host (src/utils/load.h:226, src/test_fp16.cu:295). */
/* ------------------------------------------------------------------------- */
uint16_t orc_f32_to_f16(float f)
{
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u)                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (ax > 0x7F800000u ? (0x0200u | ((ax >> 13) & 0x3FFu)) : 0u));
    if (ax >= 0x477FF000u)                       /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (ax < 0x33000001u)                        /* <= 2^-25 : rounds to zero */
        return (uint16_t)sign;
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;   /* 24-bit significand */
    uint32_t shift, half;
    if (e < -14) {                               /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));      /* 14..24 */
        half = m >> shift;
    } else {
        shift = 13;
        half = ((uint32_t)(e + 15) << 10) + ((m >> 13) & 0x3FFu);
    }
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (half & 1u))) half++;   /* carry may bump exponent: correct */
    return (uint16_t)(sign | half);
}

float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) x = sign;
        else {                                   /* subnormal: normalise */
            int s = 0;
            while (!(m & 0x400u)) { m <<= 1; s++; }
            m &= 0x3FFu;
            x = sign | ((uint32_t)(127 - 15 - s + 1) << 23) | (m << 13);
        }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e - 15 + 127) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4);
    return f;
}

/* float <-> bfloat16 (round to nearest even), the implicit conversions of the
 * reference's bf16 build (MAT_VAL_TYPE __nv_bfloat16, src/common.h:20-25; value
 * assignment at src/utils/load.h:224). */
uint16_t orc_f32_to_bf16(float f)
{
    uint32_t x; memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t lsb = (x >> 16) & 1u;
    return (uint16_t)((x + 0x7FFFu + lsb) >> 16);
}
float orc_bf16_to_f32(uint16_t h)
{
    uint32_t x = (uint32_t)h << 16; float f; memcpy(&f, &x, 4); return f;
}
void orc_f32_to_bf16_array(const float *src, uint16_t *dst, size_t n)
{ for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_bf16(src[i]); }
void orc_bf16_to_f32_array(const uint16_t *src, float *dst, size_t n)
{ for (size_t i = 0; i < n; ++i) dst[i] = orc_bf16_to_f32(src[i]); }

void orc_f32_to_f16_array(const float *src, uint16_t *dst, size_t n)
{ for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_f16(src[i]); }

void orc_f16_to_f32_array(const uint16_t *src, float *dst, size_t n)
{ for (size_t i = 0; i < n; ++i) dst[i] = orc_f16_to_f32(src[i]); }

/* ------------------------------------------------------------------------- */
/* MatrixMarket coordinate text -> CSR.  Follows src/utils/load.h:152-322.   */
/* ------------------------------------------------------------------------- */
typedef struct {
    uint32_t rows, cols, nnzs;      /* CSR_MTX, src/utils/class.h:30-37 */
    uint32_t declared_nnz;          /* the header's count before the shrink at load.h:234-238 */
    uint32_t *row_ptr;              /* rows + 1 */
    uint32_t *col_idx;              /* nnzs */
    void     *values;               /* nnzs x (2 bytes fp16 | 4 bytes fp32) */
    int       status;               /* 0 ok, 1 cannot open, 2 bad size line, 3 alloc, 4 index out of range */
} orc_csr;

typedef struct { uint32_t r, c, seq; } orc_key;

static int orc_key_cmp(const void *a, const void *b)
{
    const orc_key *x = (const orc_key *)a, *y = (const orc_key *)b;
    if (x->r != y->r) return x->r < y->r ? -1 : 1;      /* load.h:141-142 row first */
    if (x->c != y->c) return x->c < y->c ? -1 : 1;      /* load.h:144 then column   */
    /* The reference's qsort is unstable for equal (row,col); file order is kept here
       so that the oracle is deterministic.  Inputs with duplicates are ill-defined
       in the reference. */
    return x->seq < y->seq ? -1 : (x->seq > y->seq);
}

/* kind: 2 = fp16 build (USE_FP16, value rounded with RN, load.h:226),
 *       4 = fp32 storage (USE_TF32, value kept as parsed, load.h:224),
 *       3 = bf16 build (USE_BF16, value rounded with RN by the assignment, load.h:224). */
orc_csr *orc_mtx_read(const char *path, int kind)
{
    const int elem_size = kind == 4 ? 4 : 2;
    orc_csr *m = (orc_csr *)calloc(1, sizeof(orc_csr));
    if (!m) return NULL;
    FILE *f = fopen(path, "r");
    if (!f) { m->status = 1; return m; }                               /* load.h:176-180 */
    char line[1024];                                                   /* load.h:155 */
    int have = 0;
    while (fgets(line, sizeof line, f)) {                              /* load.h:183-187 */
        have = 1;
        if (line[0] != '%') break;
    }
    uint32_t rows, cols, nnz;
    if (!have || sscanf(line, "%u %u %u", &rows, &cols, &nnz) != 3) {  /* load.h:190-194 */
        fclose(f); m->status = 2; return m;
    }
    uint32_t *ri = (uint32_t *)malloc((size_t)(nnz ? nnz : 1) * 4);
    uint32_t *ci = (uint32_t *)malloc((size_t)(nnz ? nnz : 1) * 4);
    float    *vf = (float *)malloc((size_t)(nnz ? nnz : 1) * 4);
    if (!ri || !ci || !vf) { fclose(f); free(ri); free(ci); free(vf); m->status = 3; return m; }
    uint32_t count = 0;
    while (count < nnz && fgets(line, sizeof line, f)) {               /* load.h:215 */
        uint32_t r, c; float v;
        if (sscanf(line, "%u %u %f", &r, &c, &v) == 3) {               /* load.h:219 */
            ri[count] = r - 1; ci[count] = c - 1; vf[count] = v;       /* load.h:221-222 */
            count++;
        }                                                              /* other lines are skipped */
    }
    fclose(f);
    m->declared_nnz = nnz;
    nnz = count;                                                       /* load.h:234-238 */
    for (uint32_t i = 0; i < nnz; ++i)
        if (ri[i] >= rows || ci[i] >= cols) { free(ri); free(ci); free(vf); m->status = 4; return m; }

    orc_key *keys = (orc_key *)malloc((size_t)(nnz ? nnz : 1) * sizeof(orc_key));
    m->row_ptr = (uint32_t *)calloc((size_t)rows + 1, 4);
    m->col_idx = (uint32_t *)malloc((size_t)(nnz ? nnz : 1) * 4);
    m->values  = malloc((size_t)(nnz ? nnz : 1) * (size_t)elem_size);
    if (!keys || !m->row_ptr || !m->col_idx || !m->values) {
        free(keys); free(ri); free(ci); free(vf); m->status = 3; return m;
    }
    for (uint32_t i = 0; i < nnz; ++i) { keys[i].r = ri[i]; keys[i].c = ci[i]; keys[i].seq = i; }
    qsort(keys, nnz, sizeof(orc_key), orc_key_cmp);                    /* load.h:256-257 */
    for (uint32_t i = 0; i < nnz; ++i) {                               /* load.h:284-300 */
        uint32_t s = keys[i].seq;
        m->col_idx[i] = ci[s];
        if (kind == 2) ((uint16_t *)m->values)[i] = orc_f32_to_f16(vf[s]);
        else if (kind == 3) ((uint16_t *)m->values)[i] = orc_f32_to_bf16(vf[s]);
        else                ((float *)m->values)[i] = vf[s];
        m->row_ptr[ri[s] + 1]++;
    }
    for (uint32_t r = 0; r < rows; ++r) m->row_ptr[r + 1] += m->row_ptr[r];
    m->rows = rows; m->cols = cols; m->nnzs = nnz;
    free(keys); free(ri); free(ci); free(vf);
    return m;
}

void orc_csr_free(orc_csr *m)
{
    if (!m) return;
    free(m->row_ptr); free(m->col_idx); free(m->values); free(m);
}

/* Structural checks of src/utils/load.h:44-73 (validate_csr_from_coo, parts 1-2).
 * Returns the number of violations. */
int orc_csr_validate(uint32_t rows, uint32_t cols, uint32_t nnz,
                     const uint32_t *row_ptr, const uint32_t *col_idx)
{
    int bad = 0;
    if (row_ptr[0] != 0) bad++;                                        /* load.h:44-47 */
    if (row_ptr[rows] != nnz) bad++;                                   /* load.h:49-53 */
    for (uint32_t i = 0; i < rows; ++i) if (row_ptr[i] > row_ptr[i + 1]) bad++;   /* load.h:56-62 */
    for (uint32_t i = 0; i < nnz; ++i) if (col_idx[i] >= cols) bad++;  /* load.h:66-73 */
    return bad;
}

/* ------------------------------------------------------------------------- */
/* CSR -> condensed tiles without bitmap.  Follows src/utils/convert.h:146-225 */
/* ------------------------------------------------------------------------- */
static int orc_u32_cmp(const void *a, const void *b)
{
    uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
    return x < y ? -1 : (x > y);
}

/* Pass 1: sizes.  eff_windows = windows holding at least one stored entry
 * (convert.h:161-163); total_tiles = sum over them of ceil(distinct cols / CW)
 * (convert.h:178-186). */
void orc_btcf_count(uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                    uint32_t cw, uint32_t *eff_windows, uint32_t *total_tiles)
{
    uint32_t W = 0, T = 0, cap = 0; uint32_t *tmp = NULL;
    for (uint32_t r0 = 0; r0 < rows; r0 += ORC_ROW_WINDOW) {
        uint32_t r1 = r0 + ORC_ROW_WINDOW < rows ? r0 + ORC_ROW_WINDOW : rows;   /* convert.h:158 */
        uint32_t b = row_ptr[r0], e = row_ptr[r1], n = e - b;
        if (n == 0) continue;                                                     /* convert.h:162 */
        if (n > cap) { cap = n; tmp = (uint32_t *)realloc(tmp, (size_t)cap * 4); }
        memcpy(tmp, col_idx + b, (size_t)n * 4);
        qsort(tmp, n, 4, orc_u32_cmp);                                            /* convert.h:167 */
        uint32_t u = 1;
        for (uint32_t i = 1; i < n; ++i) if (tmp[i] != tmp[i - 1]) u++;          /* convert.h:169 */
        W++; T += (u + cw - 1) / cw;
    }
    free(tmp);
    *eff_windows = W; *total_tiles = T;
}

/* Pass 2: fill caller-provided arrays.
 *   rowOffset[W+1], tcA2B[T*cw], data[T*8*cw*elem_size] (zeroed here), rowIdx[W].
 * transpose != 0 selects the SPARSE_A_TRANSPOSE element order (convert.h:207-209). */
void orc_btcf_fill(uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                   const void *values, uint32_t elem_size, uint32_t cw, int transpose,
                   uint32_t *rowOffset, uint32_t *tcA2B, void *data, uint32_t *rowIdx)
{
    uint32_t W = 0, T = 0, cap = 0; uint32_t *uniq = NULL;
    rowOffset[0] = 0;                                                             /* convert.h:152 */
    const size_t tile_elems = (size_t)ORC_ROW_WINDOW * cw;
    for (uint32_t r0 = 0; r0 < rows; r0 += ORC_ROW_WINDOW) {
        uint32_t r1 = r0 + ORC_ROW_WINDOW < rows ? r0 + ORC_ROW_WINDOW : rows;
        uint32_t b = row_ptr[r0], e = row_ptr[r1], n = e - b;
        if (n == 0) continue;
        if (n > cap) { cap = n; uniq = (uint32_t *)realloc(uniq, (size_t)cap * 4); }
        memcpy(uniq, col_idx + b, (size_t)n * 4);
        qsort(uniq, n, 4, orc_u32_cmp);
        uint32_t u = 1;
        for (uint32_t i = 1; i < n; ++i) if (uniq[i] != uniq[i - 1]) uniq[u++] = uniq[i];
        uint32_t tiles = (u + cw - 1) / cw;
        uint32_t *a2b = tcA2B + (size_t)T * cw;
        for (uint32_t i = 0; i < tiles * cw; ++i) a2b[i] = i < u ? uniq[i] : ORC_IDX_MAX;   /* convert.h:178-184 */
        rowOffset[W + 1] = rowOffset[W] + tiles;                                  /* convert.h:186 */
        rowIdx[W] = r0;                                                           /* convert.h:187 */
        unsigned char *win = (unsigned char *)data + (size_t)T * tile_elems * elem_size;
        memset(win, 0, (size_t)tiles * tile_elems * elem_size);                   /* convert.h:191-193 */
        for (uint32_t r = r0; r < r1; ++r) {                                      /* convert.h:196 */
            for (uint32_t id = row_ptr[r]; id < row_ptr[r + 1]; ++id) {           /* convert.h:197 */
                uint32_t c = col_idx[id], lo = 0, hi = u;                         /* rank of c, convert.h:198 */
                while (hi - lo > 1) { uint32_t mid = (lo + hi) / 2; if (uniq[mid] <= c) lo = mid; else hi = mid; }
                uint32_t tc = lo / cw, lc = lo % cw, lr = r % ORC_ROW_WINDOW;     /* convert.h:199-201 */
                size_t off = transpose ? (size_t)lc * ORC_ROW_WINDOW + lr         /* convert.h:209 */
                                       : (size_t)lr * cw + lc;                    /* convert.h:212 */
                memcpy(win + ((size_t)tc * tile_elems + off) * elem_size,         /* convert.h:215 (later id overwrites) */
                       (const unsigned char *)values + (size_t)id * elem_size, elem_size);
            }
        }
        W++; T += tiles;
    }
    free(uniq);
}

/* ------------------------------------------------------------------------- */
/* Bitmap-compressed tiles.  Follows CSR2BTCF, src/utils/convert.h:22-139.   */
/* ------------------------------------------------------------------------- */
/* Sizes are those of orc_btcf_count (same windows and tiles, convert.h:40-58);
 * `data` holds one entry per stored CSR entry (convert.h:118,130).
 *   rowOffset[W+1], nnzOffset[T+1], tcA2B[T*cw], tcBit[T*words] (zeroed here),
 *   data[nnz*elem_size], rowIdx[W];  words = 2 for cw = 16, 1 for cw = 8
 *   (convert.h:61-66).
 * as_reference != 0: the word of bit b of tile t is t + b/64, exactly as written
 * (convert.h:83,96-101), so neighbouring 8 x 16 tiles share a word;
 * as_reference == 0: word words*t + b/64 (every tile owns its words).
 * The reference collects the entries of every tile in growing vectors
 * (convert.h:71-79,114-119) and appends them tile after tile (convert.h:122-133);
 * here the vectors are linked lists threaded through `next`. */
void orc_bitmap_fill(uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                     const void *values, uint32_t elem_size, uint32_t cw, int transpose, int as_reference,
                     uint32_t *rowOffset, uint32_t *nnzOffset, uint32_t *tcA2B, uint64_t *tcBit,
                     void *data, uint32_t *rowIdx)
{
    const uint32_t words = cw == 16 ? 2u : 1u;
    uint32_t W = 0, T = 0, cap = 0, lcap = 0;
    uint32_t *uniq = NULL, *next = NULL, *head = NULL, *tail = NULL;
    size_t out = 0;                                /* entries appended to data so far */
    uint32_t eff = 0, tot = 0;
    orc_btcf_count(rows, row_ptr, col_idx, cw, &eff, &tot);
    memset(tcBit, 0, (size_t)tot * words * 8);
    rowOffset[0] = 0;                                                             /* convert.h:29 */
    nnzOffset[0] = 0;                                                             /* convert.h:136 */
    for (uint32_t r0 = 0; r0 < rows; r0 += ORC_ROW_WINDOW) {
        uint32_t r1 = r0 + ORC_ROW_WINDOW < rows ? r0 + ORC_ROW_WINDOW : rows;    /* convert.h:34 */
        uint32_t b = row_ptr[r0], e = row_ptr[r1], n = e - b;
        if (n == 0) continue;                                                     /* convert.h:38 */
        if (n > cap) {
            cap = n;
            uniq = (uint32_t *)realloc(uniq, (size_t)cap * 4);
            next = (uint32_t *)realloc(next, (size_t)cap * 4);
        }
        memcpy(uniq, col_idx + b, (size_t)n * 4);
        qsort(uniq, n, 4, orc_u32_cmp);                                           /* convert.h:42 */
        uint32_t u = 1;
        for (uint32_t i = 1; i < n; ++i) if (uniq[i] != uniq[i - 1]) uniq[u++] = uniq[i];   /* convert.h:44 */
        uint32_t tiles = (u + cw - 1) / cw;                                       /* convert.h:51-57 */
        uint32_t *a2b = tcA2B + (size_t)T * cw;
        for (uint32_t i = 0; i < tiles * cw; ++i) a2b[i] = i < u ? uniq[i] : ORC_IDX_MAX;   /* convert.h:51-56 */
        rowOffset[W + 1] = rowOffset[W] + tiles;                                  /* convert.h:58 */
        rowIdx[W] = r0;                                                           /* convert.h:68 */
        /* one list per tile, or per tile column in the transposed order */
        uint32_t lists = transpose ? tiles * cw : tiles;
        if (lists > lcap) {
            lcap = lists;
            head = (uint32_t *)realloc(head, (size_t)lcap * 4);
            tail = (uint32_t *)realloc(tail, (size_t)lcap * 4);
        }
        for (uint32_t i = 0; i < lists; ++i) head[i] = tail[i] = ORC_IDX_MAX;
        for (uint32_t r = r0; r < r1; ++r) {                                      /* convert.h:81 */
            for (uint32_t id = row_ptr[r]; id < row_ptr[r + 1]; ++id) {           /* convert.h:82 */
                uint32_t c = col_idx[id], lo = 0, hi = u;
                while (hi - lo > 1) { uint32_t mid = (lo + hi) / 2; if (uniq[mid] <= c) lo = mid; else hi = mid; }
                uint32_t tc = lo / cw, lc = lo % cw, lr = r % ORC_ROW_WINDOW;     /* convert.h:83 */
                uint32_t bit = transpose ? lc * ORC_ROW_WINDOW + lr               /* convert.h:90 */
                                         : lr * cw + lc;                          /* convert.h:93 */
                size_t tile = (size_t)T + tc;                                     /* offset_index, convert.h:83 */
                if (words == 2) {
                    size_t base = as_reference ? tile : tile * 2;
                    if (bit < 64) tcBit[base] |= 1ull << bit;                     /* convert.h:97-98 */
                    else tcBit[base + 1] |= 1ull << (bit - 64);                   /* convert.h:99-100 */
                } else if (bit < 64) tcBit[tile] |= 1ull << bit;                  /* convert.h:104-106 */
                uint32_t list = transpose ? tc * cw + lc : tc;                    /* convert.h:112,116 */
                uint32_t k = id - b;
                next[k] = ORC_IDX_MAX;
                if (head[list] == ORC_IDX_MAX) head[list] = k; else next[tail[list]] = k;
                tail[list] = k;
            }
        }
        uint32_t per = transpose ? cw : 1u;
        for (uint32_t t = 0; t < tiles; ++t) {                                    /* convert.h:122-133 */
            for (uint32_t l = t * per; l < (t + 1) * per; ++l)
                for (uint32_t k = head[l]; k != ORC_IDX_MAX; k = next[k]) {
                    memcpy((unsigned char *)data + out * elem_size,
                           (const unsigned char *)values + ((size_t)b + k) * elem_size, elem_size);
                    out++;
                }
            nnzOffset[T + t + 1] = (uint32_t)out;                                 /* convert.h:84,135-137 */
        }
        W++; T += tiles;
    }
    free(uniq); free(next); free(head); free(tail);
}

/* ------------------------------------------------------------------------- */
/* Grouped format.  Follows BTCF2GBTCF, src/utils/convert.h:232-276.         */
/* ------------------------------------------------------------------------- */
/* Returns the number of groups; *tgl_out = max((u32)mean tiles per window,
 * min_len) (convert.h:239-243; the reference fixes min_len = 32).  Pass NULL
 * arrays to get the sizes only.  groupOffset[groups+1], groupRowIdx[groups],
 * atomic[groups]. */
uint32_t orc_group(uint32_t eff_windows, const uint32_t *rowOffset, const uint32_t *rowIdx, uint32_t min_len,
                   uint32_t *tgl_out, uint32_t *groupOffset, uint32_t *groupRowIdx, uint8_t *atomic)
{
    double sum = 0.0;
    for (uint32_t i = 0; i < eff_windows; ++i) sum += (double)(rowOffset[i + 1] - rowOffset[i]);   /* convert.h:235-239 */
    uint32_t mean = eff_windows ? (uint32_t)(sum / (double)eff_windows) : 0u;
    uint32_t tgl = mean > min_len ? mean : min_len;                               /* convert.h:243 */
    if (tgl_out) *tgl_out = tgl;
    uint32_t g = 0;
    for (uint32_t i = 0; i < eff_windows; ++i) {
        uint32_t n = rowOffset[i + 1] - rowOffset[i];
        uint32_t group_num = (n + tgl - 1) / tgl;                                 /* convert.h:249 */
        for (uint32_t j = 0; j < group_num; ++j, ++g) {
            if (!groupOffset) continue;
            groupOffset[g] = rowOffset[i] + (n + group_num - 1) / group_num * j;  /* convert.h:251 */
            groupRowIdx[g] = rowIdx[i];                                           /* convert.h:253 */
            atomic[g] = group_num == 1 ? 0 : 1;                                   /* convert.h:254-257 */
        }
    }
    if (groupOffset) groupOffset[g] = eff_windows ? rowOffset[eff_windows] : 0u;  /* convert.h:261 */
    return g;
}

/* ------------------------------------------------------------------------- */
/* SpMM oracles.  Arithmetic of src/test_fp16.cu:292-297 applied to C = A*B: */
/* products of half->float values accumulated in fp32, k (column) ascending, */
/* result rounded once to fp16 with RN (src/fp16.cu:131,167: float acc,      */
/* implicit float->__half store).                                            */
/* ------------------------------------------------------------------------- */
static int orc_threads(int req)
{
#ifdef _OPENMP
    return req > 0 ? req : omp_get_max_threads();
#else
    (void)req; return 1;
#endif
}

int orc_max_threads(void) { return orc_threads(0); }

/* C[rows x N] (fp16) = A_csr (fp16) * B[cols x N] (fp16).  absdot, when not NULL,
 * receives sum_k |a||b| per output (fp32) for error bounds in tests. */
static void orc_spmm_csr_16(int bf, uint32_t rows, uint32_t N, const uint32_t *row_ptr, const uint32_t *col_idx,
                            const uint16_t *vals, const uint16_t *B, uint16_t *C, float *absdot, int nthreads);

void orc_spmm_csr_f16(uint32_t rows, uint32_t N, const uint32_t *row_ptr, const uint32_t *col_idx,
                      const uint16_t *vals, const uint16_t *B, uint16_t *C, float *absdot, int nthreads)
{ orc_spmm_csr_16(0, rows, N, row_ptr, col_idx, vals, B, C, absdot, nthreads); }

/* Same arithmetic with bfloat16 storage (the reference's -DUSE_BF16 types). */
void orc_spmm_csr_bf16(uint32_t rows, uint32_t N, const uint32_t *row_ptr, const uint32_t *col_idx,
                       const uint16_t *vals, const uint16_t *B, uint16_t *C, float *absdot, int nthreads)
{ orc_spmm_csr_16(1, rows, N, row_ptr, col_idx, vals, B, C, absdot, nthreads); }

static void orc_spmm_csr_16(int bf, uint32_t rows, uint32_t N, const uint32_t *row_ptr, const uint32_t *col_idx,
                            const uint16_t *vals, const uint16_t *B, uint16_t *C, float *absdot, int nthreads)
{
    int nt = orc_threads(nthreads); (void)nt;
    #pragma omp parallel num_threads(nt)
    {
        float *acc = (float *)malloc((size_t)N * 4 * 2);
        float *mag = acc + N;
        #pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < (int64_t)rows; ++r) {
            for (uint32_t j = 0; j < N; ++j) { acc[j] = 0.0f; mag[j] = 0.0f; }
            for (uint32_t id = row_ptr[r]; id < row_ptr[r + 1]; ++id) {
                float a = bf ? orc_bf16_to_f32(vals[id]) : orc_f16_to_f32(vals[id]);
                const uint16_t *b = B + (size_t)col_idx[id] * N;
                if (absdot) for (uint32_t j = 0; j < N; ++j) {
                    float p = a * (bf ? orc_bf16_to_f32(b[j]) : orc_f16_to_f32(b[j])); acc[j] += p; mag[j] += fabsf(p);
                } else if (bf) for (uint32_t j = 0; j < N; ++j) acc[j] += a * orc_bf16_to_f32(b[j]);
                else for (uint32_t j = 0; j < N; ++j) acc[j] += a * orc_f16_to_f32(b[j]);
            }
            uint16_t *c = C + (size_t)r * N;
            for (uint32_t j = 0; j < N; ++j) c[j] = bf ? orc_f32_to_bf16(acc[j]) : orc_f32_to_f16(acc[j]);
            if (absdot) memcpy(absdot + (size_t)r * N, mag, (size_t)N * 4);
        }
        free(acc);
    }
}

/* fp32 storage variant (USE_TF32 build: MAT_VAL_TYPE float, src/common.h:27).
 * trunc_tf32 != 0 masks the low 13 mantissa bits of both inputs before the
 * product, which is what a tensor core does with raw fp32 bits; the reference's
 * conversion helper does not write back (src/ptx/ptx_utils.h:32-37). */
static inline float orc_tf32_trunc(float f)
{ uint32_t x; memcpy(&x, &f, 4); x &= 0xFFFFE000u; memcpy(&f, &x, 4); return f; }

void orc_spmm_csr_f32(uint32_t rows, uint32_t N, const uint32_t *row_ptr, const uint32_t *col_idx,
                      const float *vals, const float *B, float *C, float *absdot,
                      int trunc_tf32, int nthreads)
{
    int nt = orc_threads(nthreads); (void)nt;
    #pragma omp parallel for schedule(dynamic, 64) num_threads(nt)
    for (int64_t r = 0; r < (int64_t)rows; ++r) {
        float *c = C + (size_t)r * N;
        float *mg = absdot ? absdot + (size_t)r * N : NULL;
        for (uint32_t j = 0; j < N; ++j) c[j] = 0.0f;
        if (mg) for (uint32_t j = 0; j < N; ++j) mg[j] = 0.0f;
        for (uint32_t id = row_ptr[r]; id < row_ptr[r + 1]; ++id) {
            float a = trunc_tf32 ? orc_tf32_trunc(vals[id]) : vals[id];
            const float *b = B + (size_t)col_idx[id] * N;
            for (uint32_t j = 0; j < N; ++j) {
                float bv = trunc_tf32 ? orc_tf32_trunc(b[j]) : b[j];
                float p = a * bv; c[j] += p; if (mg) mg[j] += fabsf(p);
            }
        }
    }
}

/* Tile-order SpMM: the walk the reference kernel intends (src/fp16.cu:86-90,
 * 138-170): for each effective window, for each of its tiles, for each k whose
 * tcA2B entry is not IDX_MAX, every window row accumulates
 * data[t][r][k] * B[tcA2B[t][k]][:] in fp32; C[rowIdx[w]+r][:] = RN16(acc).
 * Rows outside every effective window, and nothing beyond `rows`, are written
 * as zero (the reference leaves them uninitialised; zero is the SpMM value). */
static void orc_spmm_btcf_16(int bf, uint32_t rows, uint32_t N, uint32_t eff_windows,
                             const uint32_t *rowOffset, const uint32_t *tcA2B, const uint16_t *data,
                             const uint32_t *rowIdx, const uint16_t *B, uint16_t *C);
void orc_spmm_btcf_f16(uint32_t rows, uint32_t N, uint32_t eff_windows,
                       const uint32_t *rowOffset, const uint32_t *tcA2B, const uint16_t *data,
                       const uint32_t *rowIdx, const uint16_t *B, uint16_t *C)
{ orc_spmm_btcf_16(0, rows, N, eff_windows, rowOffset, tcA2B, data, rowIdx, B, C); }
void orc_spmm_btcf_bf16(uint32_t rows, uint32_t N, uint32_t eff_windows,
                        const uint32_t *rowOffset, const uint32_t *tcA2B, const uint16_t *data,
                        const uint32_t *rowIdx, const uint16_t *B, uint16_t *C)
{ orc_spmm_btcf_16(1, rows, N, eff_windows, rowOffset, tcA2B, data, rowIdx, B, C); }

static void orc_spmm_btcf_16(int bf, uint32_t rows, uint32_t N, uint32_t eff_windows,
                             const uint32_t *rowOffset, const uint32_t *tcA2B, const uint16_t *data,
                             const uint32_t *rowIdx, const uint16_t *B, uint16_t *C)
{
    const uint32_t cw = 16;
    memset(C, 0, (size_t)rows * N * 2);
    float *acc = (float *)malloc((size_t)ORC_ROW_WINDOW * N * 4);
    for (uint32_t w = 0; w < eff_windows; ++w) {
        memset(acc, 0, (size_t)ORC_ROW_WINDOW * N * 4);
        for (uint32_t t = rowOffset[w]; t < rowOffset[w + 1]; ++t)
            for (uint32_t k = 0; k < cw; ++k) {
                uint32_t col = tcA2B[(size_t)t * cw + k];
                if (col == ORC_IDX_MAX) continue;
                const uint16_t *b = B + (size_t)col * N;
                for (uint32_t r = 0; r < ORC_ROW_WINDOW; ++r) {
                    uint16_t ab = data[((size_t)t * ORC_ROW_WINDOW + r) * cw + k];
                    float a = bf ? orc_bf16_to_f32(ab) : orc_f16_to_f32(ab);
                    float *ar = acc + (size_t)r * N;
                    if (bf) for (uint32_t j = 0; j < N; ++j) ar[j] += a * orc_bf16_to_f32(b[j]);
                    else for (uint32_t j = 0; j < N; ++j) ar[j] += a * orc_f16_to_f32(b[j]);
                }
            }
        for (uint32_t r = 0; r < ORC_ROW_WINDOW && rowIdx[w] + r < rows; ++r)
            for (uint32_t j = 0; j < N; ++j)
                C[(size_t)(rowIdx[w] + r) * N + j] = bf ? orc_f32_to_bf16(acc[(size_t)r * N + j])
                                                        : orc_f32_to_f16(acc[(size_t)r * N + j]);
    }
    free(acc);
}

void orc_spmm_btcf_f32(uint32_t rows, uint32_t N, uint32_t eff_windows, uint32_t cw,
                       const uint32_t *rowOffset, const uint32_t *tcA2B, const float *data,
                       const uint32_t *rowIdx, const float *B, float *C)
{
    memset(C, 0, (size_t)rows * N * 4);
    float *acc = (float *)malloc((size_t)ORC_ROW_WINDOW * N * 4);
    for (uint32_t w = 0; w < eff_windows; ++w) {
        memset(acc, 0, (size_t)ORC_ROW_WINDOW * N * 4);
        for (uint32_t t = rowOffset[w]; t < rowOffset[w + 1]; ++t)
            for (uint32_t k = 0; k < cw; ++k) {
                uint32_t col = tcA2B[(size_t)t * cw + k];
                if (col == ORC_IDX_MAX) continue;
                const float *b = B + (size_t)col * N;
                for (uint32_t r = 0; r < ORC_ROW_WINDOW; ++r) {
                    float a = data[((size_t)t * ORC_ROW_WINDOW + r) * cw + k];
                    float *ar = acc + (size_t)r * N;
                    for (uint32_t j = 0; j < N; ++j) ar[j] += a * b[j];
                }
            }
        for (uint32_t r = 0; r < ORC_ROW_WINDOW && rowIdx[w] + r < rows; ++r)
            memcpy(C + (size_t)(rowIdx[w] + r) * N, acc + (size_t)r * N, (size_t)N * 4);
    }
    free(acc);
}

/* ------------------------------------------------------------------------- */
/* Tile-level check arithmetic of the reference's micro-tests.               */
/* ------------------------------------------------------------------------- */
/* src/test_fp16.cu:284-297: C[i][j] = sum_k h2f(A[i*K+k]) * h2f(B[j*K+k]), both K-major. */
void orc_tile_mma_f16(const uint16_t *A, const uint16_t *B, float *C, int M, int N, int K)
{
    for (int i = 0; i < M; ++i) for (int j = 0; j < N; ++j) {
        float s = 0.0f;
        for (int k = 0; k < K; ++k) s += orc_f16_to_f32(A[i * K + k]) * orc_f16_to_f32(B[j * K + k]);
        C[i * N + j] = s;
    }
}
/* test/02.tma_and_wgmma/tma_wgmma.cu:217-230: same with fp32 inputs. */
void orc_tile_mma_f32(const float *A, const float *B, float *C, int M, int N, int K)
{
    for (int i = 0; i < M; ++i) for (int j = 0; j < N; ++j) {
        float s = 0.0f;
        for (int k = 0; k < K; ++k) s += A[i * K + k] * B[j * K + k];
        C[i * N + j] = s;
    }
}
/* src/tf32.cu:16-28 (== test/03.warp_specialized/utils.h:31-43):
 * C[r][c] += A[r*K*T + i*K + k] * B[c*K*T + i*K + k], tiles outermost. */
void orc_tile_accum_f32(const float *A, const float *B, float *C, int M, int N, int K, int T)
{
    for (int i = 0; i < M * N; ++i) C[i] = 0.0f;
    for (int i = 0; i < T; ++i)
        for (int r = 0; r < M; ++r) for (int c = 0; c < N; ++c) for (int k = 0; k < K; ++k)
            C[r * N + c] += A[r * K * T + k + i * K] * B[c * K * T + k + i * K];
}

/* Verdict of src/test_fp16.cu:302-309: fails where |e-a| / (|e| + 1e-8) > tol. */
size_t orc_verdict_rel(const float *expected, const float *actual, size_t n, float tol)
{
    size_t bad = 0;
    for (size_t i = 0; i < n; ++i) {
        float rel = fabsf(expected[i] - actual[i]) / (fabsf(expected[i]) + 1e-8f);
        if (!(rel <= tol)) bad++;
    }
    return bad;
}
/* Verdict of src/tf32.cu:37-70: relative if |ref| > 1e-6, else absolute 1e-5. */
size_t orc_verdict_rel_abs(const float *actual, const float *ref, size_t n, double tol)
{
    size_t bad = 0;
    for (size_t i = 0; i < n; ++i) {
        double err = fabs((double)actual[i] - (double)ref[i]);
        double rv = fabs((double)ref[i]);
        if (rv > 1e-6) { if (!(err / rv <= tol)) bad++; }
        else if (!(err <= 1e-5)) bad++;
    }
    return bad;
}
