/*
 * cute_oracle.c -- CPU restatement of the reference cuTeSpMM host algorithms.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists so that the
 * HIP path can be checked against an independent, serial, plain-C statement
 * of what the reference computes.  Only tests, the smoke check and the CPU
 * baseline leg of the benchmark may load it; the shipped library never does.
 *
 * Each function names the reference lines (relative to the reference root)
 * whose behaviour it restates.  The serialisation follows the shipped build
 * flags TM=16, TK=16 (compile.sh:1, inc.h:16-37).
 *
 * How each function is pinned (i.e. which independent fact a mistake here
 * would violate) is listed next to it; the checks themselves live in tests/.
 *
 *   orc_mtx_read            meta.data rows (M,K,nnz) of the shipped matrices;
 *                           closed forms for padding and symmetric expansion.
 *   orc_hrpb_build          structural invariants, dense round trip through an
 *                           independent Python decoder, the recorded first
 *                           block of ae_matrices/G67, brute force on tiny inputs.
 *   orc_partition           closed-form worked examples; tiling invariants.
 *   orc_spmm_csr/_coo       dense A.B in float64 (numpy) and scipy CSR product.
 *   orc_spmm_hrpb           equals orc_spmm_csr on the same input (exactly when
 *                           products are exactly representable).
 *   orc_check_gemm          hand-computed 4-element cases incl. skip-zero rule.
 *   parity against cuSPARSE result *bits* (spmm.cu:860-960): PARITY UNPINNED --
 *                           closed binary, no stored outputs; tolerance only.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#define ORC_TM 16u
#define ORC_TK 16u
#define ORC_BRICK_M 16u
#define ORC_BRICK_K 4u
#define ORC_BRICKS_PER_BLOCK 4u
/* word offsets inside one block record, inc.h:28-37 with TK=16 */
#define ORC_OFF_NEXT_ADDR 0u
#define ORC_OFF_COL_PTR 2u
#define ORC_OFF_PATTERN_NNZ 4u
#define ORC_OFF_NEXT_COLS 8u
#define ORC_OFF_NNZ_PREFIX 24u
#define ORC_OFF_FETCH 26u
#define ORC_OFF_NEXT_FETCH 27u
#define ORC_OFF_BITMAPS 28u
#define ORC_META_WORDS 36u
#define ORC_CHUNK_WORDS 128u

/* ------------------------------------------------------------------ */
/* MatrixMarket reader, IO.cu:10-87                                    */
/* ------------------------------------------------------------------ */

/* First integer token of a line starting at *p; advances *p. Mirrors
 * `ss >> word; stoi(word)` (IO.cu:25-28,36-39). Returns 0 if no token. */
static int orc_next_int(char **p, long *out)
{
    char *s = *p;
    while (*s == ' ' || *s == '\t' || *s == '\r' || *s == '\n') ++s;
    if (*s == '\0') return 0;
    char *e;
    long v = strtol(s, &e, 10);
    if (e == s) return 0;
    /* skip the remainder of the whitespace-delimited word (e.g. "1.5e3") */
    while (*e && *e != ' ' && *e != '\t' && *e != '\r' && *e != '\n') ++e;
    *p = e;
    *out = v;
    return 1;
}

/* Reads `path`; returns 0 on success.  Output arrays are malloc'ed.
 * IO.cu:16    symmetric iff the FIRST line contains "symmetric"
 * IO.cu:17-22 following lines starting with '%' are skipped; first other line is the size line
 * IO.cu:30-31 M, K rounded up to multiples of TM, TK
 * IO.cu:34-45 pass 1 counts entries per row (mirror for symmetric off-diagonals)
 * IO.cu:61-85 pass 2 scatters in file order; every value is 1.0f (IO.cu:68,81) */
int orc_mtx_read(const char *path, uint32_t *M_out, uint32_t *K_out, uint32_t *nnz_out,
                 uint32_t **rowPtr_out, uint32_t **cols_out, float **vals_out)
{
    FILE *f = fopen(path, "r");
    if (!f) return -1;
    size_t cap = 1 << 16;
    char *line = (char *)malloc(cap);
    if (!fgets(line, (int)cap, f)) { fclose(f); free(line); return -2; }
    int symmetric = strstr(line, "symmetric") != NULL;
    int have = 0;
    while (fgets(line, (int)cap, f)) {
        if (line[0] == '%') continue;
        have = 1;
        break;
    }
    if (!have) { fclose(f); free(line); return -3; }
    char *p = line;
    long m, k;
    if (!orc_next_int(&p, &m) || !orc_next_int(&p, &k)) { fclose(f); free(line); return -4; }
    uint32_t M = (uint32_t)(((m - 1) / ORC_TM + 1) * ORC_TM);
    uint32_t K = (uint32_t)(((k - 1) / ORC_TK + 1) * ORC_TK);
    long data_pos = ftell(f);
    uint32_t *rowPtr = (uint32_t *)calloc((size_t)M + 1, sizeof(uint32_t));
    while (fgets(line, (int)cap, f)) {
        p = line;
        long s, e;
        if (!orc_next_int(&p, &s) || !orc_next_int(&p, &e)) continue;
        rowPtr[s]++;
        if (symmetric && s != e) rowPtr[e]++;
    }
    for (uint32_t i = 0; i < M; ++i) rowPtr[i + 1] += rowPtr[i];
    uint32_t total = rowPtr[M];
    uint32_t *cols = (uint32_t *)malloc(((size_t)total + 1) * sizeof(uint32_t));
    float *vals = (float *)malloc(((size_t)total + 1) * sizeof(float));
    uint32_t *counters = (uint32_t *)calloc(M, sizeof(uint32_t));
    uint32_t nnz = 0;
    fseek(f, data_pos, SEEK_SET);
    while (fgets(line, (int)cap, f)) {
        p = line;
        long s1, e1;
        if (!orc_next_int(&p, &s1) || !orc_next_int(&p, &e1)) continue;
        uint32_t s = (uint32_t)(s1 - 1), e = (uint32_t)(e1 - 1);
        cols[rowPtr[s] + counters[s]] = e;
        vals[rowPtr[s] + counters[s]] = 1.0f;
        counters[s]++;
        nnz++;
        if (symmetric && s != e) {
            cols[rowPtr[e] + counters[e]] = s;
            vals[rowPtr[e] + counters[e]] = 1.0f;
            counters[e]++;
            nnz++;
        }
    }
    free(counters);
    free(line);
    fclose(f);
    *M_out = M; *K_out = K; *nnz_out = nnz;
    *rowPtr_out = rowPtr; *cols_out = cols; *vals_out = vals;
    return 0;
}

void orc_free(void *p) { free(p); }

/* ------------------------------------------------------------------ */
/* HRPB builder, data.cu:94-335 (serial restatement)                   */
/* ------------------------------------------------------------------ */

static int orc_cmp_u32(const void *a, const void *b)
{
    uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
    return (x > y) - (x < y);
}

/* Builds the four canonical arrays.  Preconditions as in the reference:
 * M % 16 == 0, K % 16 == 0, columns strictly increasing inside each row
 * (data.cu:204,256-258 rely on it).
 *   blockedRowPtr[P+1]   prefix of #blocks per 16-row panel   (data.cu:143,170-183)
 *   activeCols[nb*16]    per panel sorted distinct columns, zero padded (data.cu:159-160,204-210)
 *   sizePtr[nb+1]        word offset of every block record     (data.cu:294,312-322)
 *   blocksData[words]    the record stream                     (data.cu:212-296,309,323)
 * The reference builds per-thread pieces and stitches them; the stitched result
 * does not depend on the thread count, so one serial sweep states it. */
int orc_hrpb_build(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols,
                   const float *vals, uint32_t **blockedRowPtr_out, uint32_t **activeCols_out,
                   uint64_t **sizePtr_out, uint32_t **blocksData_out,
                   uint32_t *numBlocks_out, uint64_t *numWords_out)
{
    if (M % ORC_TM || K % ORC_TK) return -1;
    uint32_t P = M / ORC_TM;
    uint32_t *count_in_panel = (uint32_t *)calloc(K, sizeof(uint32_t)); /* "helper", data.cu:95,129,198 */
    uint32_t *compact = (uint32_t *)malloc((size_t)K * sizeof(uint32_t)); /* "col_map_vec", data.cu:208 */
    uint32_t *act = (uint32_t *)malloc((size_t)K * sizeof(uint32_t));
    uint32_t *blockedRowPtr = (uint32_t *)calloc((size_t)P + 1, sizeof(uint32_t));

    /* pass A (data.cu:116-149): number of blocks per panel */
    for (uint32_t p = 0; p < P; ++p) {
        uint32_t len = 0;
        for (uint32_t r = p * ORC_TM; r < (p + 1) * ORC_TM; ++r)
            for (uint32_t j = rowPtr[r]; j < rowPtr[r + 1]; ++j) {
                uint32_t c = cols[j];
                if (!count_in_panel[c]) { count_in_panel[c] = 1; act[len++] = c; }
            }
        blockedRowPtr[p + 1] = blockedRowPtr[p] + (len ? (len - 1) / ORC_TK + 1 : 0);
        for (uint32_t i = 0; i < len; ++i) count_in_panel[act[i]] = 0;
    }
    uint32_t nb = blockedRowPtr[P];
    uint32_t *activeCols = (uint32_t *)calloc((size_t)nb * ORC_TK + 1, sizeof(uint32_t));
    uint64_t *sizePtr = (uint64_t *)calloc((size_t)nb + 1, sizeof(uint64_t));
    /* upper bound of the stream: every block <= 36 + 256 values -> 3 chunks */
    uint64_t cap_words = (uint64_t)nb * 3u * ORC_CHUNK_WORDS + 1;
    uint32_t *stream = (uint32_t *)calloc(cap_words, sizeof(uint32_t));

    uint64_t addr = 0;      /* "block_addr" */
    uint64_t prev_addr = 0; /* "pre_block_addr" */
    uint32_t blk = 0;
    uint32_t cursor[ORC_TM]; /* "cp_buffer", data.cu:191,248,266 */
    for (uint32_t p = 0; p < P; ++p) {
        uint32_t row0 = p * ORC_TM;
        uint32_t len = 0;
        for (uint32_t r = 0; r < ORC_TM; ++r) {
            cursor[r] = rowPtr[row0 + r];
            for (uint32_t j = rowPtr[row0 + r]; j < rowPtr[row0 + r + 1]; ++j) {
                uint32_t c = cols[j];
                if (!count_in_panel[c]) act[len++] = c;
                count_in_panel[c]++; /* nnz of this column inside the panel, data.cu:198 */
            }
        }
        if (!len) continue;
        qsort(act, len, sizeof(uint32_t), orc_cmp_u32); /* data.cu:204 */
        for (uint32_t i = 0; i < len; ++i) {
            activeCols[(size_t)blockedRowPtr[p] * ORC_TK + i] = act[i];
            compact[act[i]] = i;
        }
        uint32_t nblk = (len - 1) / ORC_TK + 1;
        for (uint32_t b = 0; b < nblk; ++b) {
            uint32_t *rec = stream + addr;
            uint32_t nnz_blk = 0;
            for (uint32_t k = 0; k < ORC_TK; ++k) {
                if (b * ORC_TK + k < len) {
                    uint32_t c = act[b * ORC_TK + k];
                    nnz_blk += count_in_panel[c];
                    if (b) stream[prev_addr + ORC_OFF_NEXT_COLS + k] = c; /* data.cu:220-222 */
                }
            }
            uint32_t words = ((nnz_blk - 1) / 2 + 1) * 2 + ORC_META_WORDS;   /* data.cu:225 */
            uint32_t fetch = (words - 1) / ORC_CHUNK_WORDS + 1;             /* data.cu:226 */
            rec[ORC_OFF_FETCH] = fetch;
            words = fetch * ORC_CHUNK_WORDS;
            if (b) stream[prev_addr + ORC_OFF_NEXT_FETCH] = fetch;           /* data.cu:228-230 */
            uint32_t n_vals = 0;
            uint64_t col_ptr = 0;
            float *out_vals = (float *)(rec + ORC_META_WORDS);
            uint16_t prefix[ORC_BRICKS_PER_BLOCK + 1] = {0};
            for (uint32_t bc = 0; bc < ORC_BRICKS_PER_BLOCK; ++bc) {
                uint64_t bitmap = 0;
                uint32_t lo = 0, hi = 0; /* nnz in rows 0-7 / 8-15, data.cu:39 */
                int any = 0;
                for (uint32_t r = 0; r < ORC_BRICK_M; ++r) {
                    uint32_t row_end = rowPtr[row0 + r + 1];
                    while (cursor[r] < row_end) {
                        uint32_t cc = compact[cols[cursor[r]]];
                        if (cc / ORC_TK > b || (cc % ORC_TK) / ORC_BRICK_K > bc) break; /* data.cu:256-258 */
                        col_ptr |= 1ull << (bc * 4 + 0);                      /* data.cu:259-260, one brick row */
                        out_vals[n_vals++] = vals[cursor[r]];                   /* data.cu:261-263 */
                        bitmap |= 1ull << (r * ORC_BRICK_K + cc % ORC_BRICK_K); /* data.cu:36-38 */
                        if (r < 8) lo++; else hi++;
                        prefix[bc + 1]++;
                        cursor[r]++;
                        any = 1;
                    }
                }
                rec[ORC_OFF_PATTERN_NNZ + bc] = any ? (lo | (hi << 8)) : 0;  /* data.cu:270-280 */
                memcpy(rec + ORC_OFF_BITMAPS + 2 * bc, &bitmap, 8);             /* data.cu:281-285 */
            }
            for (uint32_t j = 0; j < ORC_BRICKS_PER_BLOCK; ++j) prefix[j + 1] += prefix[j];
            memcpy(rec + ORC_OFF_NNZ_PREFIX, prefix, sizeof(uint16_t) * ORC_BRICKS_PER_BLOCK); /* data.cu:290 */
            memcpy(rec + ORC_OFF_COL_PTR, &col_ptr, 8);                         /* data.cu:291 */
            prev_addr = addr;
            addr += words;
            sizePtr[blk + 1] = addr;
            blk++;
        }
        for (uint32_t i = 0; i < len; ++i) count_in_panel[act[i]] = 0;
    }
    /* next-record links (data.cu:312-317): record b holds the offset of record b+1;
     * the last record holds the stream length. */
    for (uint32_t b = 0; b < nb; ++b) {
        uint64_t next = sizePtr[b + 1];
        memcpy(stream + sizePtr[b] + ORC_OFF_NEXT_ADDR, &next, 8);
    }
    free(count_in_panel); free(compact); free(act);
    *blockedRowPtr_out = blockedRowPtr;
    *activeCols_out = activeCols;
    *sizePtr_out = sizePtr;
    *blocksData_out = stream;
    *numBlocks_out = nb;
    *numWords_out = addr;
    return 0;
}

/* ------------------------------------------------------------------ */
/* Launch partition, spmm.cu:776-812                                   */
/* ------------------------------------------------------------------ */

/* `slots` = resident thread blocks on the whole device (num_sms*num_thread_blocks
 * in spmm.cu:778-779), `nbN` = thread blocks along N (num_blocks_dimension_n).
 * Writes up to cap uint4 {start,end,panel,atomic}; returns the count. */
uint32_t orc_partition(uint32_t P, const uint32_t *blockedRowPtr, uint32_t nbN, uint32_t slots,
                       uint32_t *out4, uint32_t cap)
{
    uint32_t num_waves = (P * nbN - 1) / slots + 1;                /* spmm.cu:779 */
    uint32_t avg = blockedRowPtr[P] / P; if (avg < 1) avg = 1;      /* spmm.cu:780 */
    uint32_t n = 0;
    for (uint32_t i = 0; i < P; ++i) {
        uint32_t start = blockedRowPtr[i], end = blockedRowPtr[i + 1];
        if (start == end) continue;                                 /* spmm.cu:784-786 */
        uint32_t nblk = end - start;
        uint32_t num_loads = (nblk - 1) / avg + 1;
        uint32_t ratio = (num_loads - 1) / num_waves + 1;
        uint32_t chunk = (nblk - 1) / ratio + 1;
        if (ratio > 1) {
            for (uint32_t k = 0; k < ratio; ++k) {
                uint32_t s = start + k * chunk, e = start + (k + 1) * chunk;
                if (e > end) e = end;
                if (n < cap) { out4[4*n] = s; out4[4*n+1] = e; out4[4*n+2] = i; out4[4*n+3] = 1; }
                n++;
            }
        } else {
            if (n < cap) { out4[4*n] = start; out4[4*n+1] = end; out4[4*n+2] = i; out4[4*n+3] = 0; }
            n++;
        }
    }
    return n;
}

/* ------------------------------------------------------------------ */
/* CPU SpMM, inc.h:71-83                                               */
/* ------------------------------------------------------------------ */

/* Literal COO form: C = 0; for every nonzero in array order C[r,:] += v*B[c,:]. */
void orc_spmm_coo(const uint32_t *rows, const uint32_t *cols, const float *vals, const float *B,
                  float *C, uint32_t M, uint32_t K, uint32_t N, uint32_t nnz)
{
    (void)K;
    memset(C, 0, (size_t)M * N * sizeof(float));
    for (uint32_t i = 0; i < nnz; ++i) {
        const float *b = B + (size_t)cols[i] * N;
        float *c = C + (size_t)rows[i] * N;
        float v = vals[i];
        for (uint32_t j = 0; j < N; ++j) c[j] += v * b[j];
    }
}

/* The loop structure of inc.h:71-83 as written there: the nonzeros are walked serially and
 * the thread team is forked and joined inside, once per nonzero, over the N columns.  Same
 * sums in the same order as orc_spmm_coo; kept to show what that structure costs (one
 * fork/join per nonzero), which is why the timed CPU baseline is the row-parallel form. */
void orc_spmm_coo_inner_parallel(const uint32_t *rows, const uint32_t *cols, const float *vals, const float *B,
                                 float *C, uint32_t M, uint32_t K, uint32_t N, uint32_t nnz)
{
    (void)K;
    memset(C, 0, (size_t)M * N * sizeof(float));
    for (uint32_t i = 0; i < nnz; ++i) {
        const float *b = B + (size_t)cols[i] * N;
        float *c = C + (size_t)rows[i] * N;
        const float v = vals[i];
#pragma omp parallel for
        for (uint32_t j = 0; j < N; ++j) c[j] += v * b[j];
    }
}

/* The same sums, ordered by CSR row (each C element accumulates its row's
 * nonzeros in storage order, exactly as the COO loop does for row-major COO).
 * Rows are independent, so they may be spread over threads without changing a bit. */
void orc_spmm_csr(const uint32_t *rowPtr, const uint32_t *cols, const float *vals, const float *B,
                  float *C, uint32_t M, uint32_t N)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (uint32_t r = 0; r < M; ++r) {
        float *c = C + (size_t)r * N;
        for (uint32_t j = 0; j < N; ++j) c[j] = 0.0f;
        for (uint32_t i = rowPtr[r]; i < rowPtr[r + 1]; ++i) {
            const float *b = B + (size_t)cols[i] * N;
            float v = vals[i];
#pragma omp simd
            for (uint32_t j = 0; j < N; ++j) c[j] += v * b[j];
        }
    }
}

/* ------------------------------------------------------------------ */
/* SpMM straight from the HRPB stream, following the kernel's decode   */
/* (kernel.cu:16-29 bitmap -> operand, kernel.cu:140-141,172 traversal,*/
/*  kernel.cu:257-287 C tile placement), in fp32 instead of TF32.      */
/* ------------------------------------------------------------------ */
void orc_spmm_hrpb(uint32_t M, uint32_t N, const uint32_t *blockedRowPtr, const uint32_t *activeCols,
                   const uint64_t *sizePtr, const uint32_t *blocksData, const float *B, float *C)
{
    uint32_t P = M / ORC_TM;
    memset(C, 0, (size_t)M * N * sizeof(float));
    for (uint32_t p = 0; p < P; ++p) {
        for (uint32_t b = blockedRowPtr[p]; b < blockedRowPtr[p + 1]; ++b) {
            const uint32_t *rec = blocksData + sizePtr[b];
            const uint32_t *acols = activeCols + (size_t)b * ORC_TK;
            const float *nnzs = (const float *)(rec + ORC_META_WORDS);
            const uint16_t *prefix = (const uint16_t *)(rec + ORC_OFF_NNZ_PREFIX);
            for (uint32_t bc = 0; bc < ORC_BRICKS_PER_BLOCK; ++bc) {
                uint64_t bitmap;
                memcpy(&bitmap, rec + ORC_OFF_BITMAPS + 2 * bc, 8);
                uint32_t lo_word = (uint32_t)bitmap, hi_word = (uint32_t)(bitmap >> 32);
                uint32_t n_lo = rec[ORC_OFF_PATTERN_NNZ + bc] & 0xffu;   /* kernel.cu:24 */
                uint32_t count = prefix[bc];
                /* a "lane" owns bit `lane` of each 32-bit half: row lane/4 (+8), k lane%4 */
                for (uint32_t lane = 0; lane < 32; ++lane) {
                    uint32_t below = lane ? (0xffffffffu >> (32 - lane)) : 0u; /* kernel.cu:132 */
                    for (int half = 0; half < 2; ++half) {
                        uint32_t w = half ? hi_word : lo_word;
                        if (!((w >> lane) & 1u)) continue;
                        uint32_t idx = (uint32_t)__builtin_popcount(w & below) + (half ? n_lo : 0u);
                        float a = nnzs[count + idx];
                        uint32_t row = p * ORC_TM + lane / 4 + (half ? 8u : 0u);
                        uint32_t col = acols[bc * ORC_BRICK_K + lane % 4];
                        const float *brow = B + (size_t)col * N;
                        float *crow = C + (size_t)row * N;
                        for (uint32_t j = 0; j < N; ++j) crow[j] += a * brow[j];
                    }
                }
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* Error metric, inc.h:84-109                                          */
/* ------------------------------------------------------------------ */

/* max over i with C[i] != 0 of |C[i]-C_HOST[i]| / |C[i]|; first argument is the trusted one. */
float orc_check_gemm(const float *C, const float *C_HOST, uint32_t M, uint32_t N)
{
    float diff = 0.0f;
    uint64_t total = (uint64_t)M * N;
    for (uint64_t i = 0; i < total; ++i) {
        if (C[i] == 0.0f) continue;
        float rel = fabsf(C[i] - C_HOST[i]) / fabsf(C[i]);
        if (rel > diff) diff = rel;
    }
    return diff;
}
