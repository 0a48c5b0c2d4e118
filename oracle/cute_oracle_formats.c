/*
 * cute_oracle_formats.c -- CPU restatement of the reference's second host API family
 * (inc/SparseCoo.hpp, inc/CSR.hpp, inc/prepareBlkEll.hpp, inc/splitter.hpp, the block
 * classifier of inc/preprocess.hpp and the double-precision CPU SpMM of inc/SPMM.cuh).
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE (see cute_oracle.c).
 * Indices are signed int, dimensions are not padded, values are kept -- as in that family.
 *
 * Pins (tests/test_formats.py):
 *   orc_coo_read / orc_coo_to_csr   hand-written files; agreement with orc_mtx_read's pattern
 *                                   after sorting; scipy.io.mmread on the committed G67.mtx
 *   orc_count_blocks / orc_to_bcsr  recorded value 8750 for G67 (16x4); dense round trip
 *   orc_blocked_ell                 blockedELLToDense(preprocess(A)) == ToDense(A); H, W closed forms
 *   orc_split                       recorded G67 counters (4325 / 1875 / 33800 / 2450 / 6200);
 *                                   heavy + light = A, disjoint; brute-force tile counts
 *   orc_block_stats / orc_classify  hand-worked rows incl. the band-walk's start and end rules
 *   orc_spmm_csr_f64                float64 numpy product
 *   orc_get_stats / orc_get_anxs    dense-matrix brute force in numpy (distinct rows, columns, nonzeros
 *                                   per block and per band); closed forms (identity, full blocks,
 *                                   a single row or column per block)
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* SparseCoo<T>(path), inc/SparseCoo.hpp:91-157                        */
/* ------------------------------------------------------------------ */
typedef struct { int row, col; float val; } orc_point;

static int orc_point_cmp(const void *a, const void *b)
{
    const orc_point *x = (const orc_point *)a, *y = (const orc_point *)b;
    if (x->row != y->row) return x->row < y->row ? -1 : 1;       /* SparseCoo.hpp:35-40 */
    if (x->col != y->col) return x->col < y->col ? -1 : 1;
    return 0;
}

/* Keeps file values (1.0 when the third token is missing, SparseCoo.hpp:134-139), mirrors
 * off-diagonals of symmetric files (:144-149), sorts by (row, col) (:152).  nnz = header
 * count + mirrored entries, as the reference counts it. */
int orc_coo_read(const char *path, int *dimY, int *dimX, int *nnz_out, int **rows_out, int **cols_out, float **vals_out)
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
    int hdr_nnz = 0;
    if (sscanf(line, "%d %d %d", dimY, dimX, &hdr_nnz) != 3) { fclose(f); free(line); return -4; }
    size_t cap_pts = (size_t)hdr_nnz * 2 + 16, n = 0;
    orc_point *pts = (orc_point *)malloc(cap_pts * sizeof(orc_point));
    while (fgets(line, (int)cap, f)) {
        unsigned x, y;
        double v = 1.0;
        int got = sscanf(line, "%u %u %lf", &x, &y, &v);
        if (got < 2) continue;
        if (n + 2 > cap_pts) { cap_pts *= 2; pts = (orc_point *)realloc(pts, cap_pts * sizeof(orc_point)); }
        pts[n].row = (int)x - 1; pts[n].col = (int)y - 1; pts[n].val = (float)v; n++;
        if (symmetric && x != y) { pts[n].row = (int)y - 1; pts[n].col = (int)x - 1; pts[n].val = (float)v; n++; }
    }
    fclose(f);
    free(line);
    qsort(pts, n, sizeof(orc_point), orc_point_cmp);
    int *rows = (int *)malloc((n + 1) * sizeof(int)), *cols = (int *)malloc((n + 1) * sizeof(int));
    float *vals = (float *)malloc((n + 1) * sizeof(float));
    for (size_t i = 0; i < n; ++i) { rows[i] = pts[i].row; cols[i] = pts[i].col; vals[i] = pts[i].val; }
    free(pts);
    *nnz_out = (int)n;
    *rows_out = rows; *cols_out = cols; *vals_out = vals;
    return 0;
}

/* CSR_Matrix<T>::coo2CSR, inc/CSR.hpp:162-187 (input already sorted by (row, col)). */
void orc_coo_to_csr(int nrows, int nnz, const int *rows, const int *cols, const float *vals,
                    int *rowPtr, int *cols_out, float *vals_out)
{
    memset(rowPtr, 0, sizeof(int) * ((size_t)nrows + 1));
    for (int i = 0; i < nnz; ++i) {
        vals_out[i] = vals[i];
        cols_out[i] = cols[i];
        rowPtr[rows[i] + 1]++;
    }
    for (int i = 0; i < nrows; ++i) rowPtr[i + 1] += rowPtr[i];
}

/* csr_count_blocks, inc/CSR.hpp:728-743 */
int orc_count_blocks(int nrows, int ncols, const int *rowPtr, const int *cols, int R, int C)
{
    int nb = ncols / C + 1;
    int *mask = (int *)malloc(sizeof(int) * (size_t)nb);
    for (int i = 0; i < nb; ++i) mask[i] = -1;
    int n = 0;
    for (int i = 0; i < nrows; ++i) {
        int bi = i / R;
        for (int jj = rowPtr[i]; jj < rowPtr[i + 1]; ++jj) {
            int bj = cols[jj] / C;
            if (mask[bj] != bi) { mask[bj] = bi; n++; }
        }
    }
    free(mask);
    return n;
}

/* to_BCSR, inc/CSR.hpp:760-810.  bcsr_vals must hold nblks*R*C zeros on entry. */
void orc_to_bcsr(int nrows, int ncols, const int *rowPtr, const int *cols, const float *vals, int R, int C,
                 int *bcsr_rowPtr, int *bcsr_cols, float *bcsr_vals)
{
    int nbc = ncols / C + 1;
    float **blocks = (float **)calloc((size_t)nbc, sizeof(float *));
    int n = 0;
    bcsr_rowPtr[0] = 0;
    for (int bi = 0; bi < nrows / R; ++bi) {
        for (int r = 0; r < R; ++r) {
            int i = R * bi + r;
            for (int jj = rowPtr[i]; jj < rowPtr[i + 1]; ++jj) {
                int j = cols[jj], bj = j / C, c = j % C;
                if (!blocks[bj]) { blocks[bj] = bcsr_vals + (size_t)R * C * n; bcsr_cols[n] = bj; n++; }
                blocks[bj][C * r + c] += vals[jj];
            }
        }
        for (int jj = rowPtr[R * bi]; jj < rowPtr[R * (bi + 1)]; ++jj) blocks[cols[jj] / C] = NULL;
        bcsr_rowPtr[bi + 1] = n;
    }
    free(blocks);
}

/* ------------------------------------------------------------------ */
/* Blocked-ELL, inc/prepareBlkEll.hpp:33-183                            */
/* ------------------------------------------------------------------ */

/* Pass 1: returns height (= number of block rows that contain a row, :41-46,72) and width
 * (max distinct block columns in a block row, :75-81); a second call with ellColIdx != NULL
 * fills ellColIdx[H*W] (ascending block columns, -1 padded, :83-117) and ellValues
 * [H*B x W*B] with element (row, col) at W*B*row + EIdx*B + col%B (:145). */
void orc_blocked_ell(int nrows, int ncols, const int *rowPtr, const int *cols, const float *vals, int B,
                     int *H_out, int *W_out, int *ellColIdx, float *ellValues, int *num_blocks, int *num_elems)
{
    int H = (nrows + B - 1) / B, nbc = (ncols + B - 1) / B;
    unsigned char *seen = (unsigned char *)calloc((size_t)nbc + 1, 1);
    int W = 0, blocks = 0;
    for (int br = 0; br < H; ++br) {
        int cnt = 0;
        memset(seen, 0, (size_t)nbc + 1);
        int r1 = (br + 1) * B < nrows ? (br + 1) * B : nrows;
        for (int r = br * B; r < r1; ++r)
            for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e)
                if (!seen[cols[e] / B]) { seen[cols[e] / B] = 1; cnt++; }
        if (cnt > W) W = cnt;
        blocks += cnt;
    }
    *H_out = H; *W_out = W;
    if (num_blocks) *num_blocks = blocks;
    if (!ellColIdx) { free(seen); return; }
    for (long i = 0; i < (long)H * W; ++i) ellColIdx[i] = -1;
    memset(ellValues, 0, sizeof(float) * (size_t)H * B * (size_t)W * B);
    int elems = 0;
    for (int br = 0; br < H; ++br) {
        memset(seen, 0, (size_t)nbc + 1);
        int r1 = (br + 1) * B < nrows ? (br + 1) * B : nrows;
        for (int r = br * B; r < r1; ++r)
            for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e) seen[cols[e] / B] = 1;
        int k = 0;
        for (int bc = 0; bc < nbc; ++bc)
            if (seen[bc]) ellColIdx[(long)br * W + k++] = bc;
        for (int r = br * B; r < r1; ++r)
            for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e) {
                int bc = cols[e] / B, idx = -1;
                for (int q = 0; q < W; ++q)                       /* find_EIdx, :159-183 */
                    if (ellColIdx[(long)br * W + q] == bc) { idx = q; break; }
                ellValues[(size_t)W * B * r + (size_t)idx * B + cols[e] % B] = vals[e];
                elems++;
            }
    }
    if (num_elems) *num_elems = elems;
    free(seen);
}

/* blockedELLToDense, inc/prepareBlkEll.hpp:242-266; dense is [H*B x ncols], zero on entry */
void orc_blocked_ell_to_dense(int H, int W, int B, int ncols, const int *ellColIdx, const float *ellValues, float *dense)
{
    for (int br = 0; br < H; ++br)
        for (int bc = 0; bc < W; ++bc) {
            int actual = ellColIdx[(long)br * W + bc];
            if (actual < 0) continue;
            for (int r = br * B; r < (br + 1) * B; ++r)
                for (int c = 0; c < B; ++c)
                    dense[(size_t)r * ncols + c + (size_t)actual * B] = ellValues[(size_t)r * W * B + c + (size_t)bc * B];
        }
}

/* ------------------------------------------------------------------ */
/* Splitter, inc/splitter.hpp:34-124                                    */
/* ------------------------------------------------------------------ */

/* which[e] = 1 for elements of heavy tiles (tile nnz >= threshold), 0 for light ones (:71-80,
 * :100-112); counters[5] = total tiles, heavy tiles, heavy elems, light tiles, light elems. */
void orc_split(int nrows, int ncols, const int *rowPtr, const int *cols, int tile, int threshold,
               unsigned char *which, int *counters)
{
    int ntc = ncols / tile + 1;
    int *cnt = (int *)calloc((size_t)ntc, sizeof(int));
    memset(counters, 0, 5 * sizeof(int));
    for (int r0 = 0; r0 < nrows; r0 += tile) {
        int r1 = r0 + tile < nrows ? r0 + tile : nrows;
        for (int r = r0; r < r1; ++r)
            for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e) cnt[cols[e] / tile]++;
        for (int r = r0; r < r1; ++r)
            for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e) {
                int heavy = cnt[cols[e] / tile] >= threshold;
                which[e] = (unsigned char)heavy;
                counters[heavy ? 2 : 4]++;
            }
        for (int t = 0; t < ntc; ++t)
            if (cnt[t]) {
                counters[0]++;
                counters[cnt[t] < threshold ? 3 : 1]++;
                cnt[t] = 0;
            }
    }
    free(cnt);
}

/* ------------------------------------------------------------------ */
/* Block classifier, inc/preprocess.hpp:64-151 (band walk), :172-193 (rule) */
/* ------------------------------------------------------------------ */

/* stats[(br*nbc + bc)*3 + {0,1,2}] = {nnz, underloaded 4-wide bands, overloaded bands}.
 * The walk, per row: the "previous band" starts as band 0 with 0 nonzeros (:78-79); when the
 * band index changes, the previous band is booked as underloaded (< 2 nonzeros) or
 * overloaded (> 2) to ITS block (:87-108), every skipped band in between as underloaded
 * (:110-122); the last band of a row is never booked. */
void orc_block_stats(int nrows, int ncols, const int *rowPtr, const int *cols, int B, int *stats)
{
    int nbc = (ncols + B - 1) / B + 1, bands_per_block = B / 4;
    for (int row = 0; row < nrows; ++row) {
        int br = row / B, prev_band = 0, prev_nnz = 0;
        for (int e = rowPtr[row]; e < rowPtr[row + 1]; ++e) {
            int col = cols[e], bc = col / B, band = col / 4;
            if (band != prev_band) {
                int pb = prev_band / bands_per_block;
                if (prev_nnz < 2) stats[((size_t)br * nbc + pb) * 3 + 1]++;
                else if (prev_nnz > 2) stats[((size_t)br * nbc + pb) * 3 + 2]++;
                for (int bi = prev_band + 1; bi < band; ++bi) stats[((size_t)br * nbc + bi / bands_per_block) * 3 + 1]++;
                prev_band = band;
                prev_nnz = 1;
            } else {
                prev_nnz++;
            }
            stats[((size_t)br * nbc + bc) * 3 + 0]++;
        }
    }
}

/* 0 dense (Blocked-ELL), 1 2:4-sparse, 2 very sparse (COO); densePowerFactor = 1 (:14). */
int orc_classify(int nnz, int under, int over, int B, float deviation_threshold, float underload_dominance)
{
    (void)nnz;
    float distance = 4.0f * ((float)under + (float)over) / (float)(B * B);
    float ratio = (under + over) == 0 ? 0.0f : (float)under / (float)(under + over);
    if (distance > deviation_threshold && ratio <= underload_dominance) return 0;
    if (distance > deviation_threshold && ratio > underload_dominance) return 2;
    return 1;
}

/* sequentioal_spmm, inc/SPMM.cuh:123-187 (double precision, one C element at a time) */
void orc_spmm_csr_f64(int m, int n, const int *rowPtr, const int *cols, const double *vals, const double *B, double *C)
{
    for (int row = 0; row < m; ++row)
        for (int col = 0; col < n; ++col) {
            double sum = 0;
            for (int e = rowPtr[row]; e < rowPtr[row + 1]; ++e) sum += vals[e] * B[(size_t)n * cols[e] + col];
            C[(size_t)n * row + col] = sum;
        }
}

/* ------------------------------------------------------------------ */
/* GET_STATS and GET_ANXS, gpu_kernels.cu:1049-1186                    */
/* ------------------------------------------------------------------ */
typedef struct { unsigned key; int seg; } orc_keyseg;

static int orc_keyseg_cmp(const void *a, const void *b)
{
    const orc_keyseg *x = (const orc_keyseg *)a, *y = (const orc_keyseg *)b;
    if (x->key != y->key) return x->key < y->key ? -1 : 1;
    if (x->seg != y->seg) return x->seg < y->seg ? -1 : 1;
    return 0;
}

/* Per non-empty block (key r_blk * (ncols / blocksize) + c_blk in 32-bit unsigned arithmetic, :1064-1067, so
 * block columns beyond ncols / blocksize alias into the next block row exactly as the reference's map keys do):
 * nonzeros, distinct rows, distinct columns.  stats[0] = mean of nnz / rows, [1] = mean of nnz / columns,
 * [2] = number of blocks, [3] = mean of nnz / blocksize^2 (:1108-1136).  The reference adds the float terms
 * in hash-map order; here they are added in key order, every term rounded to float as there (:1123-1125). */
void orc_get_stats(int nrows, int ncols, const int *rowPtr, const int *cols, int blocksize, float *stats)
{
    const int nnz = rowPtr[nrows];
    const unsigned per_row = (unsigned)ncols / (unsigned)blocksize;
    orc_keyseg *by_row = (orc_keyseg *)malloc(sizeof(orc_keyseg) * (size_t)(nnz + 1));
    orc_keyseg *by_col = (orc_keyseg *)malloc(sizeof(orc_keyseg) * (size_t)(nnz + 1));
    int n = 0;
    for (int r = 0; r < nrows; ++r)
        for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e, ++n) {
            const unsigned key = (unsigned)(r / blocksize) * per_row + (unsigned)(cols[e] / blocksize);
            by_row[n].key = key; by_row[n].seg = r;
            by_col[n].key = key; by_col[n].seg = cols[e];
        }
    qsort(by_row, (size_t)n, sizeof(orc_keyseg), orc_keyseg_cmp);
    qsort(by_col, (size_t)n, sizeof(orc_keyseg), orc_keyseg_cmp);
    float anrs = 0.0f, ancs = 0.0f, dens = 0.0f;
    unsigned blocks = 0;
    for (int i = 0; i < n;) {
        int j = i, rows = 0, ccount = 0;
        while (j < n && by_row[j].key == by_row[i].key) {
            if (j == i || by_row[j].seg != by_row[j - 1].seg) rows++;
            if (j == i || by_col[j].seg != by_col[j - 1].seg) ccount++;   /* same key runs: both arrays sort by key first */
            ++j;
        }
        const int cnt = j - i;
        dens += (float)cnt / (float)(blocksize * blocksize);
        anrs += (float)cnt / (float)rows;
        ancs += (float)cnt / (float)ccount;
        blocks++;
        i = j;
    }
    free(by_row);
    free(by_col);
    stats[0] = anrs / (float)blocks;
    stats[1] = ancs / (float)blocks;
    stats[2] = (float)blocks;
    stats[3] = dens / (float)blocks;
}

/* nnz / (sum over bands of the distinct segments in the band), :1139-1186: axis != 0 takes block rows as
 * bands and columns as segments, axis == 0 block columns and rows. */
float orc_get_anxs(int nrows, const int *rowPtr, const int *cols, int blocksize, int axis)
{
    const int nnz = rowPtr[nrows];
    orc_keyseg *ks = (orc_keyseg *)malloc(sizeof(orc_keyseg) * (size_t)(nnz + 1));
    int n = 0;
    for (int r = 0; r < nrows; ++r)
        for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e, ++n) {
            ks[n].key = (unsigned)(axis ? r / blocksize : cols[e] / blocksize);
            ks[n].seg = axis ? cols[e] : r;
        }
    qsort(ks, (size_t)n, sizeof(orc_keyseg), orc_keyseg_cmp);
    int sum = 0;
    for (int i = 0; i < n; ++i)
        if (i == 0 || ks[i].key != ks[i - 1].key || ks[i].seg != ks[i - 1].seg) sum++;
    free(ks);
    return (float)(unsigned)nnz / sum;      /* (float)nnz / sum with an int sum, :1185 */
}
