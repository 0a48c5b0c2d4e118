/*
 * cutespmm.h -- C ABI of the MI355X (gfx950) brick-blocked SpMM library, libcutespmm.so.
 *
 * C = A * B with A sparse fp32 (hybrid row-panel brick format, "HRPB"), B and C dense
 * fp32 row-major.  Every entry point takes plain pointers and sizes.  Functions in the
 * "host" groups never touch the GPU; functions in the "device" groups need one.
 *
 * Each declaration cites the reference interface it stands in for (paths relative to
 * the reference tree).  All functions returning int return CUTE_OK (0) or a negative
 * cute_status; cute_status_string() names it.  No function calls exit().
 *
 * Threading: handles are thread-compatible (use one plan per host thread); there is no
 * hidden global state apart from a lazily created per-process device context.
 */
#ifndef CUTESPMM_H
#define CUTESPMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Canonical format constants (inc.h:16-37 with the shipped -DTM=16 -DTK=16). */
#define CUTE_TM 16u              /* rows per row panel                                  */
#define CUTE_TK 16u              /* active columns per block                            */
#define CUTE_BRICK_M 16u         /* brick = 16 rows x 4 active columns                  */
#define CUTE_BRICK_K 4u
#define CUTE_META_WORDS 36u      /* MetaDataSize, inc.h:36                              */
#define CUTE_CHUNK_WORDS 128u    /* block records are padded to 512-byte chunks         */
#define CUTE_TILED_HDR_WORDS 32u /* one 128-byte header line per block, device layout   */

typedef enum cute_status {
    CUTE_OK = 0,
    CUTE_ERR_IO = -1,          /* file missing / unreadable / malformed                   */
    CUTE_ERR_SHAPE = -2,       /* M or K not a multiple of 16, N == 0, size overflow      */
    CUTE_ERR_UNSORTED = -3,    /* a CSR row has unsorted or duplicate columns             */
    CUTE_ERR_RANGE = -4,       /* an index is out of range                                */
    CUTE_ERR_ARG = -5,         /* null pointer / bad enum                                 */
    CUTE_ERR_NOMEM = -6,
    CUTE_ERR_HIP = -7,         /* a HIP runtime call failed; see cute_last_hip_error()    */
    CUTE_ERR_NO_DEVICE = -8,   /* no gfx950 device visible                                */
    CUTE_ERR_FORMAT = -9,      /* a format stream failed validation                       */
    CUTE_ERR_SCRATCH = -10     /* cute_spmm_run_static: the plan needs more scratch than the static buffer holds */
} cute_status;

const char *cute_status_string(int status);
/* hipGetErrorString of the most recent failing HIP call on this thread (""), never NULL. */
const char *cute_last_hip_error(void);
void cute_free(void *p);       /* releases any array returned by this library            */

/* ------------------------------------------------------------------------------------
 * host: MatrixMarket -> CSR.                       Replaces MTX_READER (IO.cu:2-88).
 * M and K are rounded up to multiples of 16 (IO.cu:30-31); symmetric files are mirrored
 * (IO.cu:42-44,77-84); entries stay in file order inside a row (IO.cu:71-75).
 * keep_values == 0 reproduces the reference, quirk for quirk: every value 1.0f (IO.cu:68,81),
 * "symmetric" anywhere on the first line means mirror (IO.cu:16).
 * keep_values != 0 is the tolerant reader: the banner "%%MatrixMarket matrix <format> <field>
 * <symmetry>" is tokenised; values are parsed (1.0 for pattern files); skew-symmetric files are
 * mirrored with the opposite sign; "array" (dense, column-major) files are read, zeros dropped;
 * complex and hermitian files, and banners with unknown words, give CUTE_ERR_FORMAT.  A file
 * without a banner is read as the reference would.  Entries keep the reference's order.
 * ---------------------------------------------------------------------------------- */
typedef struct cute_csr {
    uint32_t M, K, nnz;
    uint32_t *rowPtr;          /* [M+1]                                                    */
    uint32_t *cols;            /* [nnz]                                                    */
    float *vals;               /* [nnz]                                                    */
} cute_csr;

int cute_mtx_read(const char *path, int keep_values, cute_csr *out);
void cute_csr_release(cute_csr *csr);
/* Sorts every row by column (stable w.r.t. values) so that it satisfies the HRPB
 * precondition; returns CUTE_ERR_UNSORTED if a row holds a duplicate column. */
int cute_csr_sort_rows(cute_csr *csr);
/* Same sort, and entries that share a (row, column) position are added up in file order; the
 * arrays shrink in place and nnz follows.  No counterpart in the reference (IO.cu keeps
 * duplicates, which HRPB's precondition, data.cu:204,256-258, then forbids). */
int cute_csr_merge_duplicates(cute_csr *csr);

/* ------------------------------------------------------------------------------------
 * host: CSR -> canonical HRPB.          Replaces HRPB::HRPB + DATASTRUCT (data.cu:80-335).
 * Output arrays are word-for-word those of the reference (record layout inc.h:28-37,
 * written at data.cu:212-296).  The CSR arrays are borrowed, as in data.cu:82-84, and
 * must outlive the object.  Preconditions are checked, not assumed: M,K multiples of 16,
 * columns strictly increasing inside each row and < K.
 * ---------------------------------------------------------------------------------- */
typedef struct cute_hrpb_host {
    uint32_t M, K;
    uint32_t numRowPanels;     /* M / 16                                                   */
    uint32_t numBlocks;        /* blockedRowPtr[numRowPanels]                              */
    uint64_t numWords;         /* length of blocksData                                     */
    uint32_t *blockedRowPtr;   /* [numRowPanels+1]                                         */
    uint32_t *activeCols;      /* [numBlocks*16]                                           */
    uint64_t *sizePtr;         /* [numBlocks+1]                                            */
    uint32_t *blocksData;      /* [numWords]                                               */
    const uint32_t *rowPtr;    /* borrowed CSR                                             */
    const uint32_t *cols;
    const float *vals;
    uint32_t nnz;
    uint32_t numBricks;        /* non-empty 16x4 bricks                                    */
} cute_hrpb_host;

int cute_hrpb_build(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols,
                    const float *vals, cute_hrpb_host *out);
void cute_hrpb_host_release(cute_hrpb_host *h);

/* ------------------------------------------------------------------------------------
 * host: binary cache of a preprocessed matrix (CSR + canonical HRPB).  No counterpart in the
 * reference, which rebuilds the format on every run (run.cu:17-20).  Versioned, checksummed;
 * cute_hrpb_load returns CUTE_ERR_FORMAT for anything that is not a complete file written by
 * cute_hrpb_save of the same version.  On success `csr` owns the CSR arrays (release with
 * cute_csr_release) and `h` borrows them and owns the four format arrays (release with
 * cute_hrpb_host_release, before the CSR).
 * ---------------------------------------------------------------------------------- */
int cute_hrpb_save(const cute_hrpb_host *h, const char *path);
int cute_hrpb_load(const char *path, cute_csr *csr, cute_hrpb_host *h);

/* ------------------------------------------------------------------------------------
 * host: canonical HRPB <-> MFMA-tiled device layout (no reference counterpart for the
 * layout itself; it re-tiles what kernel.cu:16-29 decodes per lane).  Per block one
 * 128-byte header line:
 *   words  0..15  active columns, word k*4+j = column of brick j, k-th column in brick
 *   words 16..23  four 64-bit bitmaps, bit k*16+row  <=> canonical bit row*4+k, so that
 *                 bit L is the A operand of wavefront lane L in v_mfma_f32_16x16x4_f32
 *   words 24..27  index into vals[] of each brick's first value
 *   word  28      nonzeros in the block;  words 29..31 zero
 * vals[] holds every brick's nonzeros in bitmap (lane) order.  cute_hrpb_untile()
 * inverts the mapping exactly; the pair is a bijection on valid streams.
 * ---------------------------------------------------------------------------------- */
typedef struct cute_hrpb_tiled {
    uint32_t M, K, numRowPanels, numBlocks;
    uint64_t numVals;
    uint32_t *blockedRowPtr;   /* [numRowPanels+1] copy                                    */
    uint32_t *hdr;             /* [numBlocks*32]                                           */
    float *vals;               /* [numVals]                                                */
} cute_hrpb_tiled;

int cute_hrpb_retile(const cute_hrpb_host *h, cute_hrpb_tiled *out);
int cute_hrpb_untile(const cute_hrpb_tiled *t, cute_hrpb_host *out);
void cute_hrpb_tiled_release(cute_hrpb_tiled *t);

/* ------------------------------------------------------------------------------------
 * host: quad lists, the layout of the 4x4x1 MFMA kernel.  No counterpart in the reference
 * (its kernel consumes the brick stream directly, kernel.cu:88-125); derived from the same CSR
 * input as cute_hrpb_build.  Each 4-row group of a panel has its own sorted list of active
 * columns; the four lists of a panel advance in lockstep, padded to the longest.  One group
 * of the layout is 16 (row group, column) pairs = 4 steps x 4 row groups:
 *   cols[g*16 + 4*s + rg]            column of row group rg at step s of group g
 *   vals[g*64 + 4*(4*s + rg) + i]    value of row 4*rg+i of the panel in that column, else 0
 * groupPtr[q] .. groupPtr[q+1] are the groups of row panel q.  Padding steps repeat the last
 * column of their list (column 0 for an empty list) with zero values.
 * ---------------------------------------------------------------------------------- */
typedef struct cute_quad_lists {
    uint32_t M, K, numRowPanels;   /* numRowPanels: number of list units (16-row panels, or 4-row strips)  */
    uint64_t numGroups;
    uint32_t *groupPtr;        /* [numRowPanels+1]                                         */
    uint32_t *cols;            /* [numGroups*16]                                           */
    float *vals;               /* [numGroups*64]                                           */
    uint32_t *tail;            /* [numRowPanels] pair slots in use in the unit's last group (0 if it has none) */
    uint64_t numPairs;         /* (row group, column) pairs that hold a nonzero            */
    uint32_t rowsPerList;      /* 16: four lockstep lists per panel; 4: one list per strip */
} cute_quad_lists;

int cute_quad_build(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols, const float *vals,
                    cute_quad_lists *out);
/* Size of the lockstep layout without building it: its groups and its occupied pairs (fill =
 * numPairs / (16 * numGroups)); cute_hrpb_upload uses it to choose between the two layouts. */
int cute_quad_fill(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, uint64_t *numGroups, uint64_t *numPairs);
/* One list per 4-row strip (numRowPanels = M/4), nothing padded to a neighbour: for matrices with a
 * few very long rows.  A group is 16 consecutive pairs of one strip: cols[g*16 + p],
 * vals[g*64 + 4*p + i] = value of row 4*strip+i. */
int cute_quad_build_strips(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols, const float *vals,
                           cute_quad_lists *out);
void cute_quad_release(cute_quad_lists *q);
/* Sizes of either layout without building it: per 4-row strip (there are ceil(M/4)) the length of its
 * merged column list and the number of values it stores (nonzero entries). */
int cute_quad_census(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t *stripPairs,
                     uint32_t *stripVals);
/* The device form of the lists, written directly from the CSR matrix (what cute_hrpb_upload sends): per
 * group a record of CUTE_QUAD_RECORD_WORDS words {16 columns, 64-bit mask of the occupied value slots
 * (slot 4p+i = pair p, row i), index of the group's first stored value, 0} and, in `packed`, the stored
 * (nonzero) values of all groups in slot order.  rowsPerList 16: lockstep lists, a unit is a panel;
 * 4: a unit is a strip.  groupPtr[U+1] and valBase[U] (index of each unit's first stored value) follow
 * from cute_quad_census. */
#define CUTE_QUAD_RECORD_WORDS 20u
int cute_quad_pack(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t rowsPerList,
                   const uint32_t *groupPtr, const uint64_t *valBase, uint32_t *recs, float *packed);

/* ------------------------------------------------------------------------------------
 * host: launch partition.            Replaces SPMM_TC::partition (spmm.cu:776-812).
 * Same arithmetic; the machine enters through `slots` (work items resident on the whole
 * device; num_sms*num_thread_blocks at spmm.cu:778-779) and `nbN` (work items along N).
 * out4 receives {first block, end block, panel, atomic} quadruples; returns their count
 * (which may exceed cap: call again with a larger buffer), or a negative status.
 * ---------------------------------------------------------------------------------- */
int64_t cute_partition(uint32_t numRowPanels, const uint32_t *blockedRowPtr, uint32_t nbN,
                       uint32_t slots, uint32_t *out4, uint64_t cap);
/* 1 when the fast kernels' addressing (32-bit byte offsets, rows through a 24 x 24-bit multiply) covers a
 * product of this size: M, K rows and columns, N columns of B and C, num_vals stored values, partial_rows
 * rows of partial tiles (pieces of cut panels x rows per piece); else 0, and the planner takes the
 * kernels with 64-bit offsets.  The limits stand where spmm.cu:11-101 has its per-N launch constants. */
int cute_offsets_fit(uint32_t M, uint32_t K, uint32_t N, uint64_t num_vals, uint64_t partial_rows);

/* ------------------------------------------------------------------------------------
 * host: result comparison.   Replaces check_gemm_correctness_coo (inc.h:84-109):
 * max over i with C_ref[i] != 0 of |C_ref[i]-C_test[i]| / |C_ref[i]|.
 * cute_backward_error() is the cancellation-robust companion:
 * max_ij |C_ref-C_test|_ij / sum_k |a_ik||b_kj| (0/0 counts as 0).
 * ---------------------------------------------------------------------------------- */
float cute_check_gemm_correctness(const float *C_ref, const float *C_test, uint32_t M, uint32_t N);
/* host: CPU SpMM.  Replaces spmm_coo (inc.h:71-83): C = 0, then every nonzero i in array order adds
 * vals[i] * B[cols[i],:] onto C[rows[i],:] in fp32, product and sum rounded separately.  Same bits as
 * that loop; the rows are shared out among the host threads instead of forking a team per nonzero. */
int cute_spmm_coo(const uint32_t *rows, const uint32_t *cols, const float *vals, const float *B, float *C,
                  uint32_t M, uint32_t K, uint32_t N, uint32_t NNZ);
float cute_backward_error(const uint32_t *rowPtr, const uint32_t *cols, const float *vals,
                          const float *B, const float *C_ref, const float *C_test,
                          uint32_t M, uint32_t N);

/* ------------------------------------------------------------------------------------
 * host: seeded synthetic inputs (the reference only reads .mtx files; run.cu:24-27 fills
 * B with rand()).  Counter-based generator, so values do not depend on thread count.
 *   kind 1 uniform:  M x M, `p0` distinct uniformly random columns per row, values U(-1,1)
 *   kind 2 stencil:  9-point stencil on a p0 x p0 grid, 8 on / -1 off the diagonal + U(-.01,.01)
 *   kind 3 fem:      p0 node blocks of 6x6, diagonal + ~9 neighbours within +-p1 blocks, symmetric
 *   kind 4 rmat:     2^p0 nodes, p1 edges per node, (.57,.19,.19,.05), symmetrised, +I, 1/sqrt(di dj)
 *   kind 5 banded:   M = p0 rows, p1 distinct columns per row within +-p2 of the diagonal, U(-1,1)
 * Rows come out sorted by column; M is a multiple of 16 for the stock parameters.
 * ---------------------------------------------------------------------------------- */
int cute_gen_matrix(int kind, uint64_t seed, uint32_t p0, uint32_t p1, uint32_t p2, cute_csr *out);
/* dist 0: U(0,1)   1: U(-1,1)   2: N(0,1) (Box-Muller).  Element i depends only on (seed, i). */
int cute_gen_dense(uint64_t seed, int dist, uint64_t count, float *out);

/* ------------------------------------------------------------------------------------
 * host: the reference's second API family (signed int indices, dimensions as in the file,
 * values kept).  fp32 instantiation of the templates.
 * ---------------------------------------------------------------------------------- */
typedef struct cute_coo {          /* SparseCoo<float>, inc/SparseCoo.hpp:41-388 (SoA form, :250-261) */
    int32_t dimY, dimX, nnz;       /* rows, columns, entries (header count + mirrored entries)         */
    int32_t *rows, *cols;
    float *values;
} cute_coo;

typedef struct cute_csr_i32 {      /* CSR_Matrix<float>, inc/CSR.hpp:42-51                              */
    int32_t nrows, ncols, nnz;
    int32_t *rowPtr, *cols;
    float *values;
} cute_csr_i32;

/* SparseCoo<T>(path), inc/SparseCoo.hpp:91-157: keeps values (1.0 if absent), mirrors
 * symmetric files, sorts by (row, col).  The banner is tokenised as in cute_mtx_read with
 * keep_values: skew-symmetric mirrors with the opposite sign, array files are read, complex and
 * hermitian give CUTE_ERR_FORMAT (the reference searches the line for "symmetric" only, :113). */
int cute_coo_read(const char *path, cute_coo *out);
/* Adds up entries that share a position (after a stable sort by (row, col)); nnz shrinks. */
int cute_coo_merge_duplicates(cute_coo *coo);
/* save_mtx, inc/SparseCoo.hpp:263-285 ("real general", 1-based, one entry per line). */
int cute_coo_save_mtx(const cute_coo *coo, const char *path);
void cute_coo_release(cute_coo *coo);
/* CSR_Matrix<T>::coo2CSR, inc/CSR.hpp:162-187 (sorts a copy by (row, col) first). */
int cute_coo_to_csr(const cute_coo *coo, cute_csr_i32 *out);
void cute_csr_i32_release(cute_csr_i32 *csr);
/* ToDense, inc/CSR.hpp:315-329: dense[nrows*ncols] row-major, caller-zeroed. */
int cute_csr_to_dense(const cute_csr_i32 *csr, float *dense);
/* csr_count_blocks, inc/CSR.hpp:728-743: number of non-empty R x C blocks (< 0: status). */
int64_t cute_csr_count_blocks(const cute_csr_i32 *csr, int32_t R, int32_t C);

typedef struct cute_bcsr {         /* to_BCSR outputs, inc/CSR.hpp:760-810                               */
    int32_t R, C, nrows, ncols, nblks;      /* block shape, block rows, block columns, blocks         */
    int32_t *rowPtr, *cols;                 /* [nrows+1], [nblks]                                      */
    float *values;                          /* [nblks*R*C], each block row-major                       */
} cute_bcsr;
int cute_csr_to_bcsr(const cute_csr_i32 *csr, int32_t R, int32_t C, cute_bcsr *out);
void cute_bcsr_release(cute_bcsr *b);

typedef struct cute_blocked_ell {  /* preprocess<float>, inc/prepareBlkEll.hpp:15-291                    */
    int32_t blockSize, height, width;       /* ellColIdx is [height x width]                           */
    int32_t numBlocks, numElems;
    int32_t *ellColIdx;                     /* ascending block columns per block row, -1 padded        */
    float *ellValues;                       /* [height*blockSize x width*blockSize] row-major          */
} cute_blocked_ell;
int cute_blocked_ell_build(const cute_csr_i32 *csr, int32_t blockSize, cute_blocked_ell *out);
/* blockedELLToDense, inc/prepareBlkEll.hpp:242-266: dense[height*blockSize x ncols], caller-zeroed. */
int cute_blocked_ell_to_dense(const cute_blocked_ell *e, int32_t ncols, float *dense);
void cute_blocked_ell_release(cute_blocked_ell *e);

/* Device twin and SpMM of a Blocked-ELL matrix: C[height*blockSize x N] = ELL . B[ncols x N]
 * (accumulate != 0: C += ...), fp32 MFMA on the dense blocks.  Stands where the reference's harness
 * calls cusparseSpMM on a CUSPARSE_FORMAT_BLOCKED_ELL descriptor (gpu_kernels.cu:166-223).
 * blockSize must be a multiple of 16; B and C are device pointers, 16-byte aligned. */
typedef struct cute_blocked_ell_dev cute_blocked_ell_dev;
int cute_blocked_ell_upload(const cute_blocked_ell *e, cute_blocked_ell_dev **out);
void cute_blocked_ell_dev_free(cute_blocked_ell_dev *d);
int cute_blocked_ell_spmm(const cute_blocked_ell_dev *d, const float *dB, float *dC, uint32_t N, int accumulate,
                          void *stream);

typedef struct cute_split {        /* Splitter, inc/splitter.hpp:14-187                                  */
    int32_t totalTiles, numHeavyTiles, numHeavyElems, numLightTiles, numLightElems;
    cute_coo heavy, light;                  /* tile nnz >= threshold / < threshold; CSR order kept     */
} cute_split;
int cute_splitter_split(const cute_csr_i32 *csr, int32_t tile_size, int32_t nnz_threshold, cute_split *out);
void cute_split_release(cute_split *s);

typedef struct cute_block_class {  /* one non-empty blockSize^2 block, inc/preprocess.hpp:64-193          */
    int32_t blockRow, blockCol, nnz, underloads, overloads;
    int32_t kind;                           /* 0 dense, 1 2:4-sparse, 2 very sparse                    */
} cute_block_class;
/* Band statistics (:64-151) and the classification rule (:172-193); blocks sorted by
 * (blockRow, blockCol).  *out is an array of *count entries, released with cute_free. */
int cute_classify_blocks(const cute_csr_i32 *csr, int32_t blockSize, float deviation_threshold,
                         float underload_dominance, cute_block_class **out, int64_t *count);

/* The split the classifier implies (inc/preprocess.hpp:196-283 fills three containers from it): entries of blocks
 * classified dense or 2:4-sparse are the `heavy` part, entries of very sparse blocks the `light` part; tile counters
 * count blocks.  Same containers as the Splitter's. */
int cute_split_by_class(const cute_csr_i32 *csr, int32_t blockSize, float deviation_threshold, float underload_dominance,
                        cute_split *out);

/* GET_STATS, gpu_kernels.cu:1049-1137, the features its split threshold is chosen from: over the non-empty
 * blocksize^2 blocks, stats[0] = mean of nnz / distinct rows, stats[1] = mean of nnz / distinct columns,
 * stats[2] = number of blocks, stats[3] = mean of nnz / blocksize^2.  Blocks are told apart by the reference's
 * key r_blk * (ncols / blocksize) + c_blk, so with ncols not a multiple of blocksize the last block column
 * counts into block (r_blk + 1, 0), as there.  The reference adds its float terms in hash-map order; here they
 * are added in key order (results agree to float rounding, not bit for bit).  CUTE_ERR_SHAPE where the
 * reference's 32-bit keys would wrap.  An empty matrix gives NaN means and 0 blocks, as there. */
int cute_block_stats(const cute_csr_i32 *csr, int32_t blocksize, float stats[4]);
/* GET_ANXS, gpu_kernels.cu:1139-1186: nnz / number of distinct (band, segment) pairs; axis != 0: bands are
 * block rows and segments columns, axis == 0: bands are block columns and segments rows. */
int cute_anxs(const cute_csr_i32 *csr, int32_t blocksize, int32_t axis, float *out);

/* ------------------------------------------------------------------------------------
 * device: the hybrid of the reference's earlier prototypes (inc/SPMM.cuh:2528-2933, GPU_Compute_Multi_Kernel*;
 * the 2-D variant at :2898 sends tiles with more than THRESHOLD entries to the tensor cores as dense tiles and the
 * rest to a plain kernel): a matrix split into heavy tiles, kept as a Blocked-ELL matrix and multiplied by the fp32
 * MFMA kernel, and a remainder kept as CSR and multiplied by the row kernel; both into one C.
 *   mode CUTE_HYBRID_SPLITTER    the Splitter's rule (inc/splitter.hpp:71-80): a tile_size^2 tile is heavy when it
 *                                holds at least nnz_threshold entries; nnz_threshold 0: 15 % of the tile's cells, the
 *                                break-even measured on gfx950 between this library's two kernels, and no heavy part at
 *                                all when it would hold less than 2 % of the entries.  The block statistics the
 *                                reference's harness chooses from (cute_block_stats) are reported in the info.
 *   mode CUTE_HYBRID_CLASSIFIER  the classifier's rule (inc/preprocess.hpp:172-193, cute_classify_blocks): dense and
 *                                2:4-sparse blocks are heavy, very sparse ones the remainder
 * tile_size: a multiple of 16 that divides nrows and ncols (the harness pads first, gpu_kernels.cu:1415-1430).
 * ---------------------------------------------------------------------------------- */
enum { CUTE_HYBRID_SPLITTER = 0, CUTE_HYBRID_CLASSIFIER = 1 };
typedef struct cute_hybrid_info {
    int32_t tileSize, threshold, mode;      /* threshold: the one in use (0 in classifier mode)               */
    int32_t totalTiles, heavyTiles, heavyElems, lightTiles, lightElems;
    int32_t ellHeight, ellWidth;            /* Blocked-ELL shape of the heavy part (0 x 0 when there is none)  */
    float stats[4];                         /* cute_block_stats of the whole matrix at tile_size               */
} cute_hybrid_info;
typedef struct cute_hybrid cute_hybrid;
int cute_hybrid_create(const cute_csr_i32 *csr, int32_t tile_size, int32_t nnz_threshold, int32_t mode,
                       float deviation_threshold, float underload_dominance, cute_hybrid **out);
int cute_hybrid_get_info(const cute_hybrid *h, cute_hybrid_info *out);
/* dB [ncols x N], dC [nrows x N]: device pointers, 16-byte aligned; C is overwritten.  Asynchronous on `stream`. */
int cute_hybrid_spmm(const cute_hybrid *h, const float *dB, float *dC, uint32_t N, void *stream);
void cute_hybrid_free(cute_hybrid *h);


/* sequentioal_spmm, inc/SPMM.cuh:123-187: double-precision CPU CSR SpMM; returns ms. */
float cute_sequential_spmm(const cute_csr_i32 *csr, const double *vals_f64, const double *B, double *C,
                           int32_t m, int32_t k, int32_t n);

/* ------------------------------------------------------------------------------------
 * device: upload.        Replaces the cudaMalloc/cudaMemcpy tail of DATASTRUCT
 * (data.cu:327-334) and HRPB::freeDevice (data.cu:336-339).  Uploads the CSR arrays (the row
 * kernel's input) and the one MFMA layout the planner's default rules would use for this matrix --
 * brick tiles or quad lists, or neither if every panel would go to the row kernel; a plan that asks
 * for the other layout builds it then, on the device, from the device copy of the CSR arrays.
 * ---------------------------------------------------------------------------------- */
typedef struct cute_hrpb_dev cute_hrpb_dev;
int cute_hrpb_upload(const cute_hrpb_host *h, cute_hrpb_dev **out);
/* Same, with the quad-list layout forced: 0 library's choice (lockstep lists unless they would be less
 * than 60 % full), 1 four lockstep lists per 16-row panel, 2 one list per 4-row strip. */
int cute_hrpb_upload_layout(const cute_hrpb_host *h, int quad_layout, cute_hrpb_dev **out);
/* The same from a CSR matrix that already lives on the device (an earlier kernel's output, a framework tensor):
 * the device-side counterpart of HRPB::HRPB + DATASTRUCT (data.cu:80-335; the reference builds on the host and
 * times it as "preprocessing", run.cu:17-20).  dRowPtr [M+1], dCols [nnz], dVals [nnz] are device pointers; the
 * handle keeps its own copy of them.  Preconditions are checked, not assumed: M, K multiples of 16
 * (CUTE_ERR_SHAPE), row pointers ascending from 0 to nnz and columns below K (CUTE_ERR_RANGE), columns strictly
 * increasing inside a row (CUTE_ERR_UNSORTED).  The layouts are built by kernels and equal, word for word, what
 * cute_hrpb_retile and cute_quad_pack make on the host from the same matrix; only the row pointers and per-panel
 * and per-strip counts travel to the host (the planner's statistics).  Synchronises the device. */
int cute_hrpb_upload_device_csr(uint32_t M, uint32_t K, uint32_t nnz, const uint32_t *dRowPtr, const uint32_t *dCols,
                                const float *dVals, int quad_layout, cute_hrpb_dev **out);
void cute_hrpb_dev_free(cute_hrpb_dev *d);
uint64_t cute_hrpb_dev_bytes(const cute_hrpb_dev *d); /* device bytes held */
/* Inspection: what a device handle holds.  Sizes of the layouts that have been built (0 for one that has not):
 * blocks and values of the brick tiles, groups and stored values of the quad lists, rows per list (16 or 4); and
 * host copies of them -- blockedRowPtr [M/16+1], hdr [numBlocks*32], tileVals [numTileVals], groupPtr [units+1],
 * recs [numGroups*CUTE_QUAD_RECORD_WORDS], quadVals [numQuadVals]; NULL for arrays that are not wanted.  The
 * reference keeps host and device twins of its format as public fields (data.cu:56-72). */
int cute_hrpb_dev_layout_sizes(const cute_hrpb_dev *d, uint32_t *numBlocks, uint64_t *numTileVals, uint64_t *numGroups,
                               uint64_t *numQuadVals, uint32_t *rowsPerList);
int cute_hrpb_dev_read_layouts(const cute_hrpb_dev *d, uint32_t *blockedRowPtr, uint32_t *hdr, float *tileVals,
                               uint32_t *groupPtr, uint32_t *recs, float *quadVals);

/* ------------------------------------------------------------------------------------
 * device: plan + launch.   Replaces SPMM_TC::SPMM_TC / initialize_conditions / partition
 * (spmm.cu:276-822) and SPMM_TC::run (spmm.cu:823-839).
 * ---------------------------------------------------------------------------------- */
typedef enum cute_path {
    CUTE_PATH_AUTO = 0,        /* per-panel choice between the MFMA and row kernels       */
    CUTE_PATH_BRICK = 1,       /* every panel through the MFMA kernel (see mfma_shape)    */
    CUTE_PATH_ROWS = 2         /* every panel through the wavefront-per-row kernel        */
} cute_path;

typedef enum cute_precision {
    CUTE_PREC_FP32 = 0,        /* fp32 MFMA (4x4x1 or 16x16x4), fp32 operands             */
    CUTE_PREC_BF16X3 = 1       /* brick kernel on the bf16 matrix pipeline: operands split into bf16 hi + lo in registers,
                                  three products per block, fp32 accumulation; error below 2^-16 per product.  Used where it
                                  exists (brick tiles, N a multiple of 4, 32-bit offsets), fp32 elsewhere: cute_plan_info.precision
                                  says which.  Panels the planner sends to the row kernel are always fp32.  Operands must
                                  stay inside bf16's range: a magnitude above about 3.39e38 rounds to infinity in the split, and
                                  low parts below about 1e-38 are flushed (such values keep 8 bits instead of 16). */
} cute_precision;

typedef struct cute_tunables {
    int32_t path;              /* cute_path                                               */
    int32_t precision;         /* cute_precision                                          */
    float min_reuse;           /* AUTO: panels with fewer nonzeros per B row the MFMA side would fetch go to ROWS; <=0: default (1.25) */
    uint32_t slots;            /* resident work items assumed by the partition; 0: derive from device */
    uint32_t max_chunk_blocks; /* upper bound on blocks per work item; 0: none            */
    uint32_t brick_groups;     /* 16-lane column groups per lane in the brick kernel (1 or 2); 0: default */
    uint32_t pipeline;         /* brick kernel variant: 1 rolling, 2 pipelined; 0: default (rolling)             */
    uint32_t mfma_shape;       /* MFMA kernel: 1 16x16x4 bricks, 2 4x4x1 quad lists; 0: chosen per matrix (list slots per brick) */
    uint32_t max_row_nnz;      /* AUTO: panels holding a row longer than this stay on the brick kernel; 0: default  */
    uint32_t chunk_order;      /* MFMA work items: 0 library's choice (a launch that is resident at once: dealt to the SIMDs longest
                                  first where that shortens the fullest SIMD; a larger launch whose longest item is four times the
                                  mean: long items first); 1 always in panel order; 2 always dealt; 3 always long items first */
    uint32_t operand_residency; /* where B and C are when a launch starts: 0 unknown -- planned like 1, because a product on
                                  fresh data finds its operands in HBM whatever their size; 1 from HBM (a product on data no
                                  cache holds); 2 cache-resident (a tight loop over the same operands that fit the 256 MiB
                                  Infinity Cache together; ignored when they do not).  Chooses between the MFMA kernels
                                  (and, for 1, keeps two column groups per lane in mixed plans), nothing else. */
    uint32_t hub_rows;         /* > 0 (at most 256): the quad kernel on strip lists runs as persistent work-groups that keep that many
                                  of the most referenced B rows in LDS (graphs with hub vertices); 0: off.  Ignored by other plans
                                  (cute_plan_info.hubRows says how many rows a plan stages) */
} cute_tunables;

typedef struct cute_plan_info {
    uint32_t N;
    uint32_t slabWidth;        /* columns of C per work item                              */
    uint32_t numSlabs;
    uint32_t numChunks;        /* MFMA-kernel work items along the panel axis             */
    uint32_t numAtomicChunks;  /* of which are pieces of cut panels (partial tiles, added up by a second kernel; the name dates from atomics) */
    uint32_t numBrickPanels, numRowPanelsSparse, numEmptyPanels;
    uint32_t slots;
    uint32_t precision, path;
    uint32_t mfmaShape;        /* MFMA kernel in use: 1 16x16x4 bricks, 2 4x4x1 quad lists */
    uint32_t pipeline;         /* brick kernel variant in use: 1 rolling, 2 pipelined     */
    uint32_t fusedLaunch;      /* 1: MFMA chunks and sparse rows go out as one launch     */
    uint32_t dealtChunks;      /* 1: the MFMA work items were dealt to the SIMDs by length, 2: listed long items first, 0: panel order (cute_tunables.chunk_order) */
    uint32_t partialTileKiB;   /* KiB of partial tiles the pieces of cut panels store per launch (0: no panel is cut) */
    uint32_t hubRows;          /* B rows a hub plan keeps in LDS (0: not a hub plan) */
} cute_plan_info;

typedef struct cute_spmm_plan cute_spmm_plan;
/* Plan creation copies its tables to the device with synchronous copies, gathers the quad kernels' per-item heads
 * with a small kernel on the default stream and waits for it, and -- if the plan is the first to need an MFMA
 * layout the upload did not build -- builds that layout on the device, inside the format handle (which is why the
 * handle is not const; such late builds are serialised by a lock in the handle).  Call it outside stream capture. */
int cute_spmm_plan_create(cute_hrpb_dev *d, uint32_t N, const cute_tunables *t /* may be NULL */,
                          cute_spmm_plan **out);
int cute_spmm_plan_info(const cute_spmm_plan *p, cute_plan_info *out);
void cute_spmm_plan_free(cute_spmm_plan *p);
/* dB [K x N], dC [M x N]: device pointers, row-major, 16-byte aligned.  Asynchronous on
 * `stream` (a hipStream_t, NULL = default stream).  C is fully overwritten: the caller
 * need not zero it (the reference requires cudaMemset first, run.cu:43,49).  No atomics are
 * used, so equal inputs give equal bits.  A plan whose panels were cut (numAtomicChunks > 0)
 * keeps their partial tiles in a buffer of its own: launches of ONE plan must not overlap in
 * time (same stream, or ordered by events); different plans are independent.
 * B must be finite for the MFMA kernels to give the CSR product: like the reference's kernel
 * (kernel.cu:26-27,149) they multiply a stored zero into a real B row wherever a brick or a list slot
 * has no entry, so an Inf or NaN in a B row turns into NaN in every row of C whose panel (brick kernels:
 * 16 rows; quad kernels: the 4-row group) has that column active, and one in B row 0 reaches every panel
 * that pads its last block.  Rows the planner sends to the row kernel only see the B rows they reference.
 * A caller whose B may hold Inf or NaN plans with path = CUTE_PATH_ROWS, which is exact in that sense. */
int cute_spmm_run(cute_spmm_plan *p, const float *dB, float *dC, void *stream);

/* cute_spmm_run for callers that cannot allocate device memory (code under HIP graph capture, serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels, same
 * arguments, same bits in C; the partial tiles of cut panels go to a static device array of
 * CUTE_STATIC_SCRATCH_BYTES that the library's code object carries (one copy per GPU, held until the
 * process ends) instead of the plan's own buffer.  The call launches kernels and does nothing else: no
 * hipMalloc/hipFree, no copy, no memset, no synchronisation.  A plan whose partial tiles
 * (cute_plan_info.partialTileKiB) exceed the array gives CUTE_ERR_SCRATCH, and cute_last_hip_error()
 * then names both sizes.  Every call on a GPU shares that GPU's array: calls that may overlap in time
 * on one GPU -- of any plans -- race; order them (one stream, or events).  Nothing in the array has to
 * start at zero: every piece overwrites its whole tile before the adding kernel reads it. */
#define CUTE_STATIC_SCRATCH_BYTES (32u << 20)
int cute_spmm_run_static(cute_spmm_plan *p, const float *dB, float *dC, void *stream);

/* cute_spmm_run with the partial tiles of cut panels in a buffer the caller brings (device memory, 16-byte
 * aligned, at least cute_spmm_plan_scratch_bytes(p) bytes; ignored when that is 0), so that one plan can run on
 * several streams at the same time, each call with a buffer of its own.  The reference's kernel adds the
 * pieces of a split panel into C with atomicAdd (kernel.cu:258-271) and needs no such buffer, at the price of
 * results that depend on the order of arrival.  Too small a buffer gives CUTE_ERR_SCRATCH.  Same bits in C as
 * cute_spmm_run. */
uint64_t cute_spmm_plan_scratch_bytes(const cute_spmm_plan *p);
int cute_spmm_run_scratch(cute_spmm_plan *p, const float *dB, float *dC, void *stream, void *scratch,
                          uint64_t scratch_bytes);

/* ------------------------------------------------------------------------------------
 * device: plain CSR SpMM kernels -- the fp32 CSR comparison path.  Replaces
 * GPU_CSR_cuSPARSE_NEW (spmm.cu:860-960); the three algorithms restate the simple kernels
 * of inc/SPMM.cuh (898-920 thread per element, 1061-1146 wavefront per row) and a
 * vectorised wavefront-per-row variant.
 *   alg 0: thread per (row, column)   1: wavefront per row, scalar lanes
 *   alg 2: wavefront per row, float4/float2 lanes
 * cute_csr_spmm_dev takes device pointers; cute_gpu_csr_spmm takes host pointers, copies,
 * runs one warm-up plus `iters` timed launches and returns ms per launch (< 0: -status).
 * ---------------------------------------------------------------------------------- */
int cute_csr_spmm_dev(int alg, const uint32_t *dRowPtr, const uint32_t *dCols, const float *dVals,
                      const float *dB, float *dC, uint32_t M, uint32_t N, void *stream);
float cute_gpu_csr_spmm(const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t nnz,
                        const float *hB, float *hC, uint32_t m, uint32_t k, uint32_t n, int iters, int alg);

/* device pointers of the uploaded CSR copy (for cute_csr_spmm_dev on the same matrix). */
int cute_hrpb_dev_csr(const cute_hrpb_dev *d, const uint32_t **dRowPtr, const uint32_t **dCols,
                      const float **dVals);

/* ------------------------------------------------------------------------------------
 * device: timing helper used by the drivers.  Runs `warmup` untimed and `iters` timed
 * launches of the plan on `stream`, each bracketed by HIP events on that stream; writes
 * per-launch milliseconds to ms_out[iters].
 * ---------------------------------------------------------------------------------- */
int cute_spmm_time(cute_spmm_plan *p, const float *dB, float *dC, void *stream, int warmup, int iters,
                   float *ms_out);
int cute_csr_spmm_time(int alg, const cute_hrpb_dev *d, const float *dB, float *dC, uint32_t N,
                       void *stream, int warmup, int iters, float *ms_out);

int cute_device_info(int *num_cus, int *wave_size, char *arch_name, size_t arch_cap);
/* What the planner assumes about the device: the number of XCDs it spans (8 for a whole MI355X, 256 compute units;
 * 4, 2 or 1 in the partitioned modes), compute units per XCD, its share of the Infinity Cache, and whether it
 * is the whole chip (the model of where wavefronts land, which orders work items, is used there only).  Stands
 * where spmm.cu:290-690 tabulates resident warps, blocks and SM counts per machine. */
int cute_device_layout(int *num_xcds, int *cus_per_xcd, uint64_t *cache_bytes, int *whole_chip);

#ifdef __cplusplus
}
#endif
#endif /* CUTESPMM_H */
