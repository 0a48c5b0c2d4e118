// gfx950 device kernels of libcutespmm.
//
//   hrpb_brick_f32_rolling   one wavefront per (row-panel chunk, N slab) over the brick tiles; every non-empty
//                    16x4 brick is one v_mfma_f32_16x16x4_f32 A operand taken straight from the lane-order
//                    bitmap; B rows are gathered in the MFMA B-operand layout (16 lanes read one contiguous
//                    row segment), so no LDS transpose is needed.  One operand set, refilled behind the MFMAs.
//   hrpb_brick_f32   the same work with two whole operand sets in flight and 64-bit addressing (operands
//                    beyond the 32-bit offsets of the rolling variant).
//   hrpb_brick_bf16x3   the brick tiles on the bf16 matrix pipeline: operands split into bf16 high and low
//                    parts in registers, three v_mfma_f32_16x16x16_bf16 per block and 16 columns.
//   hrpb_quad_f32    quad lists: v_mfma_f32_4x4x1_16B_f32 over 16 (row group, column) pairs at a time, so
//                    only occupied 4-row column pieces cost matrix time.
//   csr_rows_batched one lane group per CSR row, lanes span N, 8 (col, val) pairs in flight; the kernel
//                    for panels with too little reuse for the matrix cores.
//   hrpb_quad_rows_f32 / hrpb_brick_rows_f32   MFMA work items and sparse rows of a mixed plan in one launch.
//   reduce_partials  adds up the partial tiles of panels that were cut, in chunk order (no atomics).
//   blocked_ell_f32  fp32 MFMA over the dense blocks of a Blocked-ELL matrix.
//   csr_rows / csr_thread_per_element / csr_wave_scalar   the simple CSR comparison kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cutespmm.h"

namespace cute_dev {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

template <int VEC> struct Vec;
template <> struct Vec<1> { typedef float type; };
template <> struct Vec<2> { typedef f32x2 type; };
template <> struct Vec<4> { typedef f32x4 type; };

template <int VEC> __device__ __forceinline__ float vec_get(const typename Vec<VEC>::type &v, int i) { return v[i]; }
template <> __device__ __forceinline__ float vec_get<1>(const float &v, int) { return v; }
template <int VEC> __device__ __forceinline__ void vec_set(typename Vec<VEC>::type &v, int i, float x) { v[i] = x; }
template <> __device__ __forceinline__ void vec_set<1>(float &v, int, float x) { v = x; }

constexpr int kWaveSize = 64;
constexpr int kWavesPerGroup = 4;
constexpr int kHdrWords = 32;
constexpr int kNumXcd = 8;
constexpr int kQuadRecordWords = CUTE_QUAD_RECORD_WORDS;   // device record of one quad-list group: 16 columns, mask lo/hi, first value, pad
constexpr int kQuadHeadWords = 32;     // quad kernels, per chunk: descriptor (4 words), first group's record, padding to 128 bytes

// Work-groups are handed to the 8 XCDs round-robin; this maps the hardware id to a
// logical id such that each XCD walks one contiguous range of logical ids (neighbouring
// row panels share B rows, which then stay in that XCD's L2).
__device__ __forceinline__ uint32_t xcd_contiguous_id(uint32_t bid, uint32_t groups_per_xcd)
{
    return (bid % kNumXcd) * groups_per_xcd + bid / kNumXcd;
}

// The same idea with ranges of unequal length (balanced by work, not by count): XCD x owns the
// logical blocks [first[x], first[x+1]); the launch has kNumXcd * (longest range) blocks.
struct XcdRanges {
    uint32_t first[kNumXcd + 1];
};

__device__ __forceinline__ bool xcd_range_id(const XcdRanges &r, uint32_t bid, uint32_t &logical)
{
    const uint32_t x = bid % kNumXcd;
    logical = r.first[x] + bid / kNumXcd;
    return logical < r.first[x + 1];
}

struct BlockHeader {          // one 128-byte header line as a wavefront sees it
    uint64_t bitmap[4];       // wave-uniform (scalar loads)
    uint32_t voff[4];         // wave-uniform
    uint4 cols;               // per lane: the (lane/16)-th active column of bricks 0..3
};

template <int VEC, int NG>
struct BlockOperands {
    float a[4];                                   // value at (brick offset + lane rank), before masking
    uint64_t bitmap[4];                           // wave-uniform: lane L is a nonzero iff bit L
    typename Vec<VEC>::type b[4][NG];             // B operand vectors per brick and column group
};

__device__ __forceinline__ BlockHeader load_header(const uint32_t *__restrict__ hdr, uint32_t blk, uint32_t lane)
{
    const uint32_t *h = hdr + size_t(blk) * kHdrWords;
    BlockHeader r;
    r.cols = reinterpret_cast<const uint4 *>(h)[lane >> 4];
    const uint64_t *bm = reinterpret_cast<const uint64_t *>(h + 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) r.bitmap[j] = bm[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) r.voff[j] = h[24 + j];
    return r;
}

// Issues every load of one block without a branch: bricks that consist of padding only
// have an all-zero bitmap and padding columns point at B row 0, so they contribute
// 0 * B[0][.] (B must be finite, as in the reference, kernel.cu:26-27,149).  vals[] is
// padded by one wavefront of floats so that the unconditional A load never leaves it.
template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void load_operands(BlockOperands<VEC, NG> &o, const BlockHeader &hd,
                                              const float *__restrict__ vals, const float *__restrict__ B,
                                              uint32_t N, uint32_t col0, uint32_t lane)
{
    typedef typename Vec<VEC>::type V;
    const uint32_t cols[4] = {hd.cols.x, hd.cols.y, hd.cols.z, hd.cols.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint64_t bm = hd.bitmap[j];
        const uint32_t below = __builtin_amdgcn_mbcnt_hi(uint32_t(bm >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(bm), 0u));
        o.a[j] = vals[hd.voff[j] + below];       // masked when consumed, so nothing waits here
        o.bitmap[j] = bm;
        const float *brow = B + size_t(cols[j]) * N;
#pragma unroll
        for (int ng = 0; ng < NG; ++ng) {
            // lanes beyond column N re-read the row's last VEC columns (N is a multiple of VEC) and store nothing:
            // a branch around the load would split the pipeline's basic blocks
            const uint32_t c = col0 + uint32_t(ng) * 16u * VEC;
            o.b[j][ng] = *reinterpret_cast<const V *>(brow + ((FULL || c < N) ? c : N - VEC));
        }
    }
}

template <int VEC, int NG>
__device__ __forceinline__ void mfma_block(const BlockOperands<VEC, NG> &o, f32x4 (&acc)[NG][VEC], uint32_t lane)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = ((o.bitmap[j] >> lane) & 1ull) ? o.a[j] : 0.0f;
#pragma unroll
        for (int ng = 0; ng < NG; ++ng)
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vec_get<VEC>(o.b[j][ng], v), acc[ng][v], 0, 0, 0);
    }
}

// chunks[i] = {first block, end block, row panel, piece}.  piece = 0: the chunk is its panel's only one and
// stores the C tile; piece = k > 0: the panel is cut, and this chunk stores its partial tile as "panel" k-1
// of the partials matrix (same row pitch as C), which reduce_partials adds up afterwards.  A work item is (chunk, slab);
// slab s covers columns [s*16*VEC*NG, (s+1)*16*VEC*NG).  Lane L = 16*g + j owns, inside
// column group ng, the VEC consecutive columns starting at s*slab + ng*16*VEC + j*VEC;
// MFMA tile v of that group therefore holds the columns {.. + j*VEC + v}, and after the
// MFMA lane L holds rows 4g..4g+3 of exactly those VEC columns -> one vector store per row.
// FULL: N is a multiple of the slab width, so no column guard is compiled in.
struct BrickItem {
    uint32_t start, end, panel, piece, col0;
    bool valid;
};

// The launch is a 2-D grid: x walks the chunks (kWavesPerGroup per work-group, remapped so that
// each XCD owns a contiguous range), y is the slab.  gridDim.x is a multiple of the XCD count,
// so the slabs of one chunk run on the same XCD and share its B rows in that L2.
template <int VEC, int NG>
__device__ __forceinline__ BrickItem brick_item(const uint4 *__restrict__ chunks, uint32_t num_chunks,
                                                uint32_t groups_per_xcd, uint32_t lane, uint32_t block_x, uint32_t block_y)
{
    BrickItem it;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const uint32_t chunk = xcd_contiguous_id(block_x, groups_per_xcd) * kWavesPerGroup + wave;
    it.valid = chunk < num_chunks;
    if (!it.valid) return it;
    const uint4 ck = chunks[chunk];
    it.start = __builtin_amdgcn_readfirstlane(ck.x);
    it.end = __builtin_amdgcn_readfirstlane(ck.y);
    it.panel = __builtin_amdgcn_readfirstlane(ck.z);
    it.piece = __builtin_amdgcn_readfirstlane(ck.w);
    it.col0 = block_y * (16u * VEC * NG) + (lane & 15u) * VEC;
    return it;
}

template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void brick_store(const BrickItem &it, const f32x4 (&acc)[NG][VEC], float *__restrict__ C,
                                            float *__restrict__ partials, uint32_t N, uint32_t lane)
{
    typedef typename Vec<VEC>::type V;
    float *out_base = it.piece ? partials : C;
    const uint32_t row0 = (it.piece ? it.piece - 1u : it.panel) * 16u + (lane >> 4) * 4u;
#pragma unroll
    for (int ng = 0; ng < NG; ++ng) {
        const uint32_t c = it.col0 + uint32_t(ng) * 16u * VEC;
        if (!FULL && c >= N) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float *dst = out_base + size_t(row0 + r) * N + c;
            V out;
#pragma unroll
            for (int v = 0; v < VEC; ++v) vec_set<VEC>(out, v, acc[ng][v][r]);
            __builtin_nontemporal_store(out, reinterpret_cast<V *>(dst));   // not read again by this launch: keep it out of the L2
        }
    }
}

// Variant "pipelined": two operand sets per wavefront ping-pong, so a wavefront overlaps its
// own loads with its own MFMAs.  Best when work items are long (many blocks per chunk) and
// few wavefronts fit per SIMD anyway.
template <int VEC, int NG, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup) void hrpb_brick_f32(
    const uint4 *__restrict__ chunks, uint32_t num_chunks, uint32_t groups_per_xcd,
    const uint32_t *__restrict__ hdr, const float *__restrict__ vals, const float *__restrict__ B,
    float *__restrict__ C, float *__restrict__ partials, uint32_t N)
{
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const BrickItem it = brick_item<VEC, NG>(chunks, num_chunks, groups_per_xcd, lane, blockIdx.x, blockIdx.y);
    if (!it.valid) return;
    const uint32_t end = it.end, col0 = it.col0;

    f32x4 acc[NG][VEC];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[ng][v] = f32x4(0.0f);

    // Software pipeline, unrolled by two so that the operand sets ping-pong without copies:
    // header lines run two blocks ahead of the MFMAs, operand loads one block ahead.  The
    // steady-state loop is a single basic block (every prefetch in it is in range), so the
    // scheduling barriers really keep each load group ahead of the MFMAs that hide it.
    BlockOperands<VEC, NG> opA, opB;
    BlockHeader hd, hn;
    uint32_t blk = it.start;
    if (blk < end) {
        hd = load_header(hdr, blk, lane);
        if (blk + 1 < end) hn = load_header(hdr, blk + 1, lane);
        load_operands<VEC, NG, FULL>(opA, hd, vals, B, N, col0, lane);
        hd = hn;
    }
    // Inside a stage the next header line is requested before the operand loads: loads
    // return in order, so the later wait for that header then leaves the operand loads in flight.
    while (blk + 4 <= end) {          // opA holds block blk, hd the header of blk+1
        hn = load_header(hdr, blk + 2, lane);
        __builtin_amdgcn_sched_barrier(0);
        load_operands<VEC, NG, FULL>(opB, hd, vals, B, N, col0, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opA, acc, lane);
        __builtin_amdgcn_sched_barrier(0);
        hd = load_header(hdr, blk + 3, lane);
        __builtin_amdgcn_sched_barrier(0);
        load_operands<VEC, NG, FULL>(opA, hn, vals, B, N, col0, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opB, acc, lane);
        __builtin_amdgcn_sched_barrier(0);
        blk += 2;
    }
    const uint32_t rem = end - blk;   // 0 (empty chunk), 1, 2 or 3 blocks left; opA/hd as above
    if (rem == 1) {
        mfma_block<VEC, NG>(opA, acc, lane);
    } else if (rem == 2) {
        load_operands<VEC, NG, FULL>(opB, hd, vals, B, N, col0, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opA, acc, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opB, acc, lane);
    } else if (rem == 3) {
        hn = load_header(hdr, blk + 2, lane);
        __builtin_amdgcn_sched_barrier(0);
        load_operands<VEC, NG, FULL>(opB, hd, vals, B, N, col0, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opA, acc, lane);
        __builtin_amdgcn_sched_barrier(0);
        load_operands<VEC, NG, FULL>(opA, hn, vals, B, N, col0, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opB, acc, lane);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block<VEC, NG>(opA, acc, lane);
    }
    brick_store<VEC, NG, FULL>(it, acc, C, partials, N, lane);
}

// One brick's loads -- the unit of the rolling pipeline below -- written for a SIMD whose
// matrix and vector instructions share one issue stream (on gfx950 an fp32 MFMA of one
// wavefront and the vector ALU work of another do not overlap), so every vector instruction
// saved is time saved:
//   * the A value is fetched already masked: lanes whose bitmap bit is clear read the zero
//     stored behind the values (the bitmap itself, a scalar register pair, is the select mask);
//   * the brick's value offset rides in the addend of the lane-rank count;
//   * both addresses are 32-bit byte offsets from a scalar base (the planner checks that B and
//     the value array are smaller than 4 GiB and that column * row pitch fits 24 x 24 bits).
struct BrickOperands {
    float a;
    f32x4 b;
};

struct LeanHeader {           // like BlockHeader, plus nothing: kept separate so the scalar parts stay scalar
    uint64_t bitmap[4];
    uint32_t voff[4];
    u32x4 cols;
};

__device__ __forceinline__ LeanHeader load_lean_header(const uint32_t *__restrict__ hdr, uint32_t blk, uint32_t lane)
{
    const uint32_t *h = hdr + size_t(blk) * kHdrWords;
    LeanHeader r;
    r.cols = *reinterpret_cast<const u32x4 *>(h + (lane >> 4) * 4u);
    const uint64_t *bm = reinterpret_cast<const uint64_t *>(h + 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) r.bitmap[j] = bm[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) r.voff[j] = h[24 + j];
    return r;
}

// col_offs[ng]: byte offset inside a B row of the lane's VEC columns in column group ng.  When N is not a multiple of
// the slab width, the lanes of the last slab that stand beyond column N point at the row's last VEC columns instead
// (N is a multiple of VEC): they load valid memory, compute values nobody stores, and the loop keeps the one basic
// block per iteration that its pipeline needs -- a branch around those loads cost 29 % (N = 192 against N = 256).
template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void brick_column_offsets(uint32_t (&col_offs)[NG], uint32_t col0, uint32_t N)
{
#pragma unroll
    for (int ng = 0; ng < NG; ++ng) {
        const uint32_t c = col0 + uint32_t(ng) * 16u * VEC;
        col_offs[ng] = ((FULL || c < N) ? c : N - VEC) * 4u;
    }
}

template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void load_brick_lean(typename Vec<VEC>::type (&b_out)[NG], float &a_out, int j,
                                                const LeanHeader &hd, const float *__restrict__ vals,
                                                uint32_t zero_index, const float *__restrict__ B, uint32_t row_pitch,
                                                const uint32_t (&col_offs)[NG])
{
    typedef typename Vec<VEC>::type V;
    const uint64_t bm = hd.bitmap[j];
    const uint32_t rank = __builtin_amdgcn_mbcnt_hi(uint32_t(bm >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(bm), hd.voff[j]));
    const uint32_t aoff = (__builtin_amdgcn_inverse_ballot_w64(bm) ? rank : zero_index) * 4u;
    a_out = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(vals) + aoff);
    const uint32_t row = __umul24(hd.cols[j], row_pitch);
    if constexpr (FULL) {       // one address, the column groups at constant offsets from it
        const char *brow = reinterpret_cast<const char *>(B) + (row + col_offs[0]);
#pragma unroll
        for (int ng = 0; ng < NG; ++ng) b_out[ng] = *reinterpret_cast<const V *>(brow + ng * 64 * VEC);
    } else {
#pragma unroll
        for (int ng = 0; ng < NG; ++ng)
            b_out[ng] = *reinterpret_cast<const V *>(reinterpret_cast<const char *>(B) + (row + col_offs[ng]));
    }
}

// C tile of one item, addressed like the loads: 32-bit byte offsets from a scalar base.
template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void brick_store_lean(const BrickItem &it, const f32x4 (&acc)[NG][VEC], float *__restrict__ C,
                                                 float *__restrict__ partials, uint32_t N, uint32_t lane)
{
    typedef typename Vec<VEC>::type V;
    char *out_base = reinterpret_cast<char *>(it.piece ? partials : C);
    const uint32_t row0 = (it.piece ? it.piece - 1u : it.panel) * 16u + (lane >> 4) * 4u;
#pragma unroll
    for (int ng = 0; ng < NG; ++ng) {
        const uint32_t c = it.col0 + uint32_t(ng) * 16u * VEC;
        if (!FULL && c >= N) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t off = __umul24(row0 + r, N * 4u) + c * 4u;
            V out;
#pragma unroll
            for (int v = 0; v < VEC; ++v) vec_set<VEC>(out, v, acc[ng][v][r]);
            __builtin_nontemporal_store(out, reinterpret_cast<V *>(out_base + off));   // not read again by this launch
        }
    }
}

// Variant "rolling": ONE operand set per wavefront, refilled brick by brick -- as soon as the
// MFMAs of brick j of block i are issued, the loads of brick j of block i+1 go out into the
// same registers.  Loads are therefore always in flight behind the MFMAs, and the register
// budget is small enough that a launch of short panels is resident as a whole.  Padding-only
// bricks skip their MFMAs.  NG = 2 lets one wavefront cover two column groups, which halves the
// header traffic and shares the A-side index arithmetic between them.
template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void brick_rolling_body(uint32_t block_x, uint32_t block_y, const uint4 *__restrict__ chunks,
                                                   uint32_t num_chunks, uint32_t groups_per_xcd,
                                                   const uint32_t *__restrict__ hdr, const float *__restrict__ vals,
                                                   uint32_t zero_index, const float *__restrict__ B, float *__restrict__ C,
                                                   float *__restrict__ partials, uint32_t N)
{
    typedef typename Vec<VEC>::type V;
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const BrickItem it = brick_item<VEC, NG>(chunks, num_chunks, groups_per_xcd, lane, block_x, block_y);
    if (!it.valid) return;
    const uint32_t end = it.end;
    const uint32_t row_pitch = N * 4u;
    uint32_t col_offs[NG];
    brick_column_offsets<VEC, NG, FULL>(col_offs, it.col0, N);

    f32x4 acc[NG][VEC];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[ng][v] = f32x4(0.0f);

    uint32_t blk = it.start;
    if (blk < end) {
        V b[4][NG];
        float a[4];
        uint64_t bitmap[4];
        LeanHeader h1, h2;
        {
            const LeanHeader h0 = load_lean_header(hdr, blk, lane);
            h1 = load_lean_header(hdr, min(blk + 1, end - 1), lane);
            // h1's load must be complete before the loop is entered.  The wait in front of its first use in
            // the loop is compiled once for both ways into the loop; were the load still in flight here (the
            // compiler would sink it behind the operand loads below), that wait would allow only two younger
            // loads and would drain the whole operand set on every iteration.  Waiting here costs nothing:
            // the operand addresses below need h0, which was requested together with h1.
            asm volatile("" ::"v"(h1.cols[0]), "v"(h1.cols[1]), "v"(h1.cols[2]), "v"(h1.cols[3]));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                load_brick_lean<VEC, NG, FULL>(b[j], a[j], j, h0, vals, zero_index, B, row_pitch, col_offs);
                bitmap[j] = h0.bitmap[j];
            }
        }
        // One basic block per iteration and a scheduling fence after every group, so the order
        // "MFMAs of brick j, then the loads that refill brick j" survives instruction scheduling.
        // Only the last block of a panel can hold padding-only bricks; it is peeled below.
        for (; blk + 1 < end; ++blk) {       // a/b hold block blk, h1 the header line of blk+1
            h2 = load_lean_header(hdr, min(blk + 2, end - 1), lane);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int ng = 0; ng < NG; ++ng)
#pragma unroll
                    for (int v = 0; v < VEC; ++v)
                        acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], vec_get<VEC>(b[j][ng], v), acc[ng][v], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                load_brick_lean<VEC, NG, FULL>(b[j], a[j], j, h1, vals, zero_index, B, row_pitch, col_offs);
                bitmap[j] = h1.bitmap[j];
                __builtin_amdgcn_sched_barrier(0);
            }
            h1 = h2;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (bitmap[j] == 0) continue;     // wave-uniform: a brick made of padding columns only
#pragma unroll
            for (int ng = 0; ng < NG; ++ng)
#pragma unroll
                for (int v = 0; v < VEC; ++v)
                    acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], vec_get<VEC>(b[j][ng], v), acc[ng][v], 0, 0, 0);
        }
    }
    brick_store_lean<VEC, NG, FULL>(it, acc, C, partials, N, lane);
}

template <int VEC, int NG, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup, (NG == 1 ? 8 : 4)) void hrpb_brick_f32_rolling(
    const uint4 *__restrict__ chunks, uint32_t num_chunks, uint32_t groups_per_xcd, const uint32_t *__restrict__ hdr,
    const float *__restrict__ vals, uint32_t zero_index, const float *__restrict__ B, float *__restrict__ C,
    float *__restrict__ partials, uint32_t N)
{
    brick_rolling_body<VEC, NG, FULL>(blockIdx.x, blockIdx.y, chunks, num_chunks, groups_per_xcd, hdr, vals, zero_index, B, C,
                                      partials, N);
}

// ---------------------------------------------------------------------------------------
// Reduced-precision brick kernel: the same tiles, loads and C layout as the rolling fp32 kernel, but the
// products run on the bf16 matrix pipeline.  Every fp32 operand x is split in registers into two bf16
// numbers, hi = bf16(x) and lo = bf16(x - hi) (round to nearest; x - hi is exact in fp32), and a block
// contributes  A_hi.B_hi + A_lo.B_hi + A_hi.B_lo  -- three v_mfma_f32_16x16x16_bf16 with fp32
// accumulation.  What is dropped (A_lo.B_lo and the rounding of the lo parts) is below 2^-16 of each
// product.  One such instruction spans the 16 active columns of a whole block: k slot 4g+i of lane
// group g is column g of brick i, which is exactly what lane group g of the fp32 kernel fetches for
// brick i -- so the block header, the masked A fetch through the lane-order bitmaps and the B gathers are
// those of the fp32 kernel unchanged, and only the arithmetic between the loads differs.  An fp32 block
// costs 4 bricks x 32 cycles per 16 columns on the matrix pipeline, this one 3 x 16; the split costs
// three vector instructions per B value, which (unlike next to fp32 MFMAs) overlap with bf16 MFMAs.
// ---------------------------------------------------------------------------------------
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// hi and lo parts of four fp32 values as two packed bf16 quadruples
__device__ __forceinline__ void split_bf16x4(float x0, float x1, float x2, float x3, s16x4 &hi, s16x4 &lo)
{
    const uint32_t h01 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){x0, x1}, bf16x2));
    const uint32_t h23 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){x2, x3}, bf16x2));
    const float r0 = x0 - __uint_as_float(h01 << 16), r1 = x1 - __uint_as_float(h01 & 0xffff0000u);
    const float r2 = x2 - __uint_as_float(h23 << 16), r3 = x3 - __uint_as_float(h23 & 0xffff0000u);
    const uint32_t l01 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){r0, r1}, bf16x2));
    const uint32_t l23 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){r2, r3}, bf16x2));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    hi = __builtin_bit_cast(s16x4, (u32x2){h01, h23});
    lo = __builtin_bit_cast(s16x4, (u32x2){l01, l23});
}

template <int NG>
struct Bf16Operands {
    s16x4 a_hi, a_lo;
    s16x4 b_hi[NG][4], b_lo[NG][4];
};

template <int NG>
__device__ __forceinline__ void split_block(Bf16Operands<NG> &o, const float (&a)[4], const f32x4 (&b)[4][NG])
{
    split_bf16x4(a[0], a[1], a[2], a[3], o.a_hi, o.a_lo);
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < 4; ++v) split_bf16x4(b[0][ng][v], b[1][ng][v], b[2][ng][v], b[3][ng][v], o.b_hi[ng][v], o.b_lo[ng][v]);
}

template <int NG>
__device__ __forceinline__ void mfma_block_bf16x3(const Bf16Operands<NG> &o, f32x4 (&acc)[NG][4])
{
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(o.a_hi, o.b_hi[ng][v], acc[ng][v], 0, 0, 0);
            acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(o.a_lo, o.b_hi[ng][v], acc[ng][v], 0, 0, 0);
            acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(o.a_hi, o.b_lo[ng][v], acc[ng][v], 0, 0, 0);
        }
}

template <int NG, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup, (NG == 1 ? 6 : 4)) void hrpb_brick_bf16x3(
    const uint4 *__restrict__ chunks, uint32_t num_chunks, uint32_t groups_per_xcd, const uint32_t *__restrict__ hdr,
    const float *__restrict__ vals, uint32_t zero_index, const float *__restrict__ B, float *__restrict__ C,
    float *__restrict__ partials, uint32_t N)
{
    constexpr int VEC = 4;
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const BrickItem it = brick_item<VEC, NG>(chunks, num_chunks, groups_per_xcd, lane, blockIdx.x, blockIdx.y);
    if (!it.valid) return;
    const uint32_t end = it.end;
    const uint32_t row_pitch = N * 4u;
    uint32_t col_offs[NG];
    brick_column_offsets<VEC, NG, FULL>(col_offs, it.col0, N);

    f32x4 acc[NG][VEC];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[ng][v] = f32x4(0.0f);

    uint32_t blk = it.start;
    if (blk < end) {
        f32x4 b[4][NG];
        float a[4];
        LeanHeader h1;
        {
            const LeanHeader h0 = load_lean_header(hdr, blk, lane);
            h1 = load_lean_header(hdr, min(blk + 1, end - 1), lane);
            asm volatile("" ::"v"(h1.cols[0]), "v"(h1.cols[1]), "v"(h1.cols[2]), "v"(h1.cols[3]));   // as in the fp32 kernel
#pragma unroll
            for (int j = 0; j < 4; ++j) load_brick_lean<VEC, NG, FULL>(b[j], a[j], j, h0, vals, zero_index, B, row_pitch, col_offs);
        }
        Bf16Operands<NG> o;
        // per block: split what has arrived, ask for the next block into the same registers, multiply
        for (; blk + 1 < end; ++blk) {       // a/b hold block blk, h1 the header line of blk+1
            const LeanHeader h2 = load_lean_header(hdr, min(blk + 2, end - 1), lane);
            __builtin_amdgcn_sched_barrier(0);
            split_block<NG>(o, a, b);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 4; ++j) load_brick_lean<VEC, NG, FULL>(b[j], a[j], j, h1, vals, zero_index, B, row_pitch, col_offs);
            __builtin_amdgcn_sched_barrier(0);
            mfma_block_bf16x3<NG>(o, acc);
            __builtin_amdgcn_sched_barrier(0);
            h1 = h2;
        }
        split_block<NG>(o, a, b);
        mfma_block_bf16x3<NG>(o, acc);
    }
    brick_store_lean<VEC, NG, FULL>(it, acc, C, partials, N, lane);
}

// ---------------------------------------------------------------------------------------
// Quad kernel: v_mfma_f32_4x4x1_16B_f32 over the quad lists (see cute_quad_lists).
//
// With cbsz = 4 the instruction takes the four A values of lanes 4p..4p+3 (abid = p), and
// multiplies them into all 64 B lanes: D[i][lane] += A[4p+i] * B[lane].  One instruction is
// therefore "one column of one 4-row group times 64 output columns" -- 8 cycles of the SIMD
// instead of the 36 a 16x16x4 tile costs, and a panel only pays for the (row group, column)
// pairs that hold a nonzero.
//
// Lane L owns output column slab*64 + L of all 16 rows: acc[rg][i] is row 4*rg+i.  A group's
// 64 values are one coalesced dword per lane and ARE the A register (lane 4p+i = pair p, row i);
// its 16 columns are wave-uniform (scalar registers); its 16 B operands are one dword per lane
// each, a contiguous 256-byte piece of a B row.  Two operand sets roll: as soon as the MFMA of
// pair p is issued, B operand p of the group after next is requested into the same register.
//
// chunks[i] = {first group, end group, row panel (or 4-row strip), piece} (piece as for the brick kernels); launch: x walks
// the chunks, y the slabs.  STRIPS: one list per 4-row strip (cute_quad_build_strips) instead of four
// lockstep lists per panel; the instruction stream is the same, only the accumulators mean something else.
// Addresses are 32-bit byte offsets from scalar bases; the planner checks the sizes.
// ---------------------------------------------------------------------------------------
template <int P>
__device__ __forceinline__ void quad_mfma(float a, float b, f32x4 (&acc)[4])
{
    acc[P & 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, acc[P & 3], 4, P, 0);
}

// HUB: the column words of the records a hub plan reads may name a slot of the work-group's LDS table of hub
// rows instead of a B row (kHubFlag | slot): that operand then comes out of LDS (see hrpb_quad_hub_f32).
constexpr uint32_t kHubFlag = 0x80000000u;

template <bool HUB>
__device__ __forceinline__ float quad_load_b(const float *__restrict__ B, uint32_t col, uint32_t row_pitch, uint32_t col_off,
                                             const float *hub)
{
    if (HUB && (col & kHubFlag))        // wave-uniform: the column is a scalar
        return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(hub) + ((col & 0x00ffffffu) * (kWaveSize * 4u) + (threadIdx.x & (kWaveSize - 1)) * 4u));
    return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(B) + (__umul24(col, row_pitch) + col_off));
}

template <bool FULL, bool STRIPS, bool HUB>
__device__ __forceinline__ void quad_chunk(uint32_t chunk, uint32_t block_y, const uint32_t *__restrict__ heads,
                                           const uint32_t *__restrict__ qrecs, const float *__restrict__ qvals, uint32_t zero_index,
                                           const float *__restrict__ B, float *__restrict__ C, float *__restrict__ partials,
                                           uint32_t N, const float *hub);

template <bool FULL, bool STRIPS>
__device__ __forceinline__ void quad_body(uint32_t block_x, uint32_t block_y, const uint32_t *__restrict__ heads,
                                          uint32_t num_chunks, uint32_t groups_per_xcd, const uint32_t *__restrict__ qrecs,
                                          const float *__restrict__ qvals, uint32_t zero_index,
                                          const float *__restrict__ B, float *__restrict__ C,
                                          float *__restrict__ partials, uint32_t N)
{
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const uint32_t chunk = xcd_contiguous_id(block_x, groups_per_xcd) * kWavesPerGroup + wave;
    if (chunk >= num_chunks) return;
    quad_chunk<FULL, STRIPS, false>(chunk, block_y, heads, qrecs, qvals, zero_index, B, C, partials, N, nullptr);
}

template <bool FULL, bool STRIPS, bool HUB>
__device__ __forceinline__ void quad_chunk(uint32_t chunk, uint32_t block_y, const uint32_t *__restrict__ heads,
                                           const uint32_t *__restrict__ qrecs, const float *__restrict__ qvals, uint32_t zero_index,
                                           const float *__restrict__ B, float *__restrict__ C, float *__restrict__ partials,
                                           uint32_t N, const float *hub)
{
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    // One entry of kQuadHeadWords per chunk: its descriptor and, behind it, the record of its first group, so
    // that the first B rows can be requested after one scalar fetch instead of two dependent ones.
    const uint32_t *head = heads + size_t(chunk) * kQuadHeadWords;
    uint32_t g = head[0];
    const uint32_t g_end = head[1];
    const uint32_t panel = head[2];
    const uint32_t piece = head[3];
    uint32_t head_rec[kQuadRecordWords];
#pragma unroll
    for (int p = 0; p < kQuadRecordWords; ++p) head_rec[p] = head[4 + p];
    // one wait for the whole entry: the compiler would otherwise sink the later words to their first use
    asm volatile("" ::"s"(head_rec[11]), "s"(head_rec[12]), "s"(head_rec[15]), "s"(head_rec[16]), "s"(head_rec[17]), "s"(head_rec[18]));

    const uint32_t n = block_y * kWaveSize + lane;
    const bool live = FULL || n < N;
    const uint32_t row_pitch = N * 4u;
    const uint32_t col_off = (live ? n : N - 1u) * 4u;      // dead lanes re-read the last column and store nothing

    f32x4 acc[4];
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) acc[rg] = f32x4(0.0f);

    if (g < g_end) {
        // Two operand sets, so every B operand is requested two groups before its MFMA: set 0 holds
        // group g, set 1 group g+1 (or a harmless re-read of the last group when there is none).
        float b0[16], b1[16], a0, a1;
        // records of the groups being requested (scalar registers): 16 columns, the 64-bit occupancy mask of
        // the group's 64 value slots and the position of its first stored value
        uint32_t ca[kQuadRecordWords], cb[kQuadRecordWords];
        const uint32_t last = g_end - 1u;
        auto fetch_cols = [&](uint32_t (&c)[kQuadRecordWords], uint32_t grp) {
            const uint32_t *src = qrecs + size_t(min(grp, last)) * kQuadRecordWords;
#pragma unroll
            for (int p = 0; p < kQuadRecordWords; ++p) c[p] = src[p];
        };
        // only occupied slots are stored: lane L's value sits (number of occupied slots below L) behind the
        // group's first one; an empty slot reads the zero kept behind the last value
        auto fetch_a = [&](const uint32_t (&c)[kQuadRecordWords]) {
            const uint64_t mask = (uint64_t(c[17]) << 32) | c[16];
            const uint32_t rank = __builtin_amdgcn_mbcnt_hi(c[17], __builtin_amdgcn_mbcnt_lo(c[16], c[18]));
            const uint32_t off = (__builtin_amdgcn_inverse_ballot_w64(mask) ? rank : zero_index) * 4u;
            return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(qvals) + off);
        };
#pragma unroll
        for (int p = 0; p < kQuadRecordWords; ++p) ca[p] = head_rec[p];
        fetch_cols(cb, g + 1);
        a0 = fetch_a(ca);
        a1 = fetch_a(cb);
#pragma unroll
        for (int p = 0; p < 16; ++p) b0[p] = quad_load_b<HUB>(B, ca[p], row_pitch, col_off, hub);
#pragma unroll
        for (int p = 0; p < 16; ++p) b1[p] = quad_load_b<HUB>(B, cb[p], row_pitch, col_off, hub);
#define CUTE_QUAD_ROLL(P, A, BSET, COLS)                          \
    quad_mfma<P>(A, BSET[P], acc);                                \
    __builtin_amdgcn_sched_barrier(0);                            \
    BSET[P] = quad_load_b<HUB>(B, COLS[P], row_pitch, col_off, hub); \
    __builtin_amdgcn_sched_barrier(0);
#define CUTE_QUAD_ROLL_REST(A, BSET, COLS)                                                                 \
    CUTE_QUAD_ROLL(1, A, BSET, COLS) CUTE_QUAD_ROLL(2, A, BSET, COLS)                                      \
    CUTE_QUAD_ROLL(3, A, BSET, COLS) CUTE_QUAD_ROLL(4, A, BSET, COLS) CUTE_QUAD_ROLL(5, A, BSET, COLS)    \
    CUTE_QUAD_ROLL(6, A, BSET, COLS) CUTE_QUAD_ROLL(7, A, BSET, COLS) CUTE_QUAD_ROLL(8, A, BSET, COLS)    \
    CUTE_QUAD_ROLL(9, A, BSET, COLS) CUTE_QUAD_ROLL(10, A, BSET, COLS) CUTE_QUAD_ROLL(11, A, BSET, COLS)  \
    CUTE_QUAD_ROLL(12, A, BSET, COLS) CUTE_QUAD_ROLL(13, A, BSET, COLS) CUTE_QUAD_ROLL(14, A, BSET, COLS) \
    CUTE_QUAD_ROLL(15, A, BSET, COLS)
#define CUTE_QUAD_MFMA16(A, BSET)                                                                          \
    quad_mfma<0>(A, BSET[0], acc);   quad_mfma<1>(A, BSET[1], acc);   quad_mfma<2>(A, BSET[2], acc);       \
    quad_mfma<3>(A, BSET[3], acc);   quad_mfma<4>(A, BSET[4], acc);   quad_mfma<5>(A, BSET[5], acc);       \
    quad_mfma<6>(A, BSET[6], acc);   quad_mfma<7>(A, BSET[7], acc);   quad_mfma<8>(A, BSET[8], acc);       \
    quad_mfma<9>(A, BSET[9], acc);   quad_mfma<10>(A, BSET[10], acc); quad_mfma<11>(A, BSET[11], acc);     \
    quad_mfma<12>(A, BSET[12], acc); quad_mfma<13>(A, BSET[13], acc); quad_mfma<14>(A, BSET[14], acc);     \
    quad_mfma<15>(A, BSET[15], acc);
        fetch_cols(ca, g + 2);
        while (g + 2 < g_end) {              // groups g, g+1 and g+2 exist
            // group g from set 0; set 0 is refilled with group g+2.  The other column list is
            // asked for right after this one's first use (where it is waited for), so that wait
            // never covers a fetch just issued; it is first used 15 pairs later.
            const float a0n = fetch_a(ca);
            __builtin_amdgcn_sched_barrier(0);
            CUTE_QUAD_ROLL(0, a0, b0, ca)
            fetch_cols(cb, g + 3);
            __builtin_amdgcn_sched_barrier(0);
            CUTE_QUAD_ROLL_REST(a0, b0, ca)
            a0 = a0n;
            // group g+1 from set 1; set 1 is refilled with group g+3 (clamped to the last one)
            const float a1n = fetch_a(cb);
            __builtin_amdgcn_sched_barrier(0);
            CUTE_QUAD_ROLL(0, a1, b1, cb)
            fetch_cols(ca, g + 4);
            __builtin_amdgcn_sched_barrier(0);
            CUTE_QUAD_ROLL_REST(a1, b1, cb)
            a1 = a1n;
            g += 2;
        }
        CUTE_QUAD_MFMA16(a0, b0)
        if (g + 1 < g_end) { CUTE_QUAD_MFMA16(a1, b1) }
#undef CUTE_QUAD_ROLL
#undef CUTE_QUAD_ROLL_REST
#undef CUTE_QUAD_MFMA16
    }
    if (live) {
        // a cut panel's chunk stores its tile into the partials matrix instead (rows (piece-1)*16.., same pitch)
        char *out_base = reinterpret_cast<char *>(piece ? partials : C);
        const uint32_t out_unit = piece ? piece - 1u : panel;
        if (STRIPS) {
            // all 16 pairs of a group belong to one 4-row strip; the four accumulators only break
            // the dependency chain and are summed here
            const f32x4 sum = (acc[0] + acc[1]) + (acc[2] + acc[3]);
            uint32_t off = __umul24(out_unit * 4u, row_pitch) + n * 4u;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                __builtin_nontemporal_store(sum[i], reinterpret_cast<float *>(out_base + off));
                off += row_pitch;
            }
        } else {
            uint32_t off = __umul24(out_unit * 16u, row_pitch) + n * 4u;
#pragma unroll
            for (int rg = 0; rg < 4; ++rg)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // not read again by this launch: keep it out of the L2
                    __builtin_nontemporal_store(acc[rg][i], reinterpret_cast<float *>(out_base + off));
                    off += row_pitch;
                }
        }
    }
}

template <bool FULL, bool STRIPS>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup, 8) void hrpb_quad_f32(
    const uint32_t *__restrict__ heads, uint32_t num_chunks, uint32_t groups_per_xcd, const uint32_t *__restrict__ qrecs,
    const float *__restrict__ qvals, uint32_t zero_index, const float *__restrict__ B, float *__restrict__ C,
    float *__restrict__ partials, uint32_t N)
{
    quad_body<FULL, STRIPS>(blockIdx.x, blockIdx.y, heads, num_chunks, groups_per_xcd, qrecs, qvals, zero_index, B, C,
                            partials, N);
}

// ---------------------------------------------------------------------------------------
// The quad kernel with the most referenced B rows staged in LDS (the reference stages the B rows of a block in
// shared memory for the warps of its thread block, kernel.cu:123-124,143-164; here what is staged is what many
// work items share: the rows of hub columns).  A work-group of sixteen wavefronts copies, once, the 64-column
// pieces of `num_hub` hub rows of its slab into LDS (num_hub * 256 bytes) and then stays: its wavefronts walk the
// chunk list with a stride of the whole launch, so the table is filled once per work-group, not once per chunk.
// A column word of the plan's records that carries kHubFlag names a slot of that table, and the operand is an
// LDS read instead of a gather through the vector memory path.  Strip lists only (graphs with hub vertices).
// ---------------------------------------------------------------------------------------
constexpr int kHubWaves = 16;

template <bool FULL>
__global__ __launch_bounds__(kWaveSize *kHubWaves) void hrpb_quad_hub_f32(
    const uint32_t *__restrict__ heads, uint32_t num_chunks, const uint32_t *__restrict__ qrecs, const float *__restrict__ qvals,
    uint32_t zero_index, const uint32_t *__restrict__ hub_rows, uint32_t num_hub, const float *__restrict__ B,
    float *__restrict__ C, float *__restrict__ partials, uint32_t N)
{
    extern __shared__ float hub[];
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const uint32_t n = blockIdx.y * kWaveSize + lane;
    for (uint32_t h = wave; h < num_hub; h += kHubWaves)
        hub[h * kWaveSize + lane] = (FULL || n < N) ? B[size_t(hub_rows[h]) * N + n] : 0.0f;
    __syncthreads();
    // consecutive chunks of the list (longest first) go to different work-groups
    const uint32_t stride = gridDim.x * kHubWaves;
    for (uint32_t chunk = wave * gridDim.x + blockIdx.x; chunk < num_chunks; chunk += stride)
        quad_chunk<FULL, true, true>(chunk, blockIdx.y, heads, qrecs, qvals, zero_index, B, C, partials, N, hub);
}

// ---------------------------------------------------------------------------------------
// Blocked-ELL SpMM (the format of inc/prepareBlkEll.hpp): dense blockSize x blockSize blocks,
// ellColIdx[height x width] block-column ids (ascending, -1 padded), ellValues row-major
// [height*blockSize x width*blockSize].  One wavefront per (16-row strip, slab of 16*VEC columns).
// A 16x16 tile of A is one 16-byte load per lane: lane (row = L%16, q = L/16) holds
// A[row][4q..4q+3].  MFMA number e of the tile takes element e of that vector, i.e. k index
// 4q+e from lane group q -- so lane group q fetches B rows 4q+e, e = 0..3, itself, and no
// cross-lane move is needed.  Accumulator layout and the column interleave that gives every
// lane VEC consecutive C columns are those of the brick kernel.
// ACCUMULATE: C += A.B (for the heavy part of a split matrix), else C = A.B.
// ---------------------------------------------------------------------------------------
constexpr int kEllDepth = 3;

template <int VEC, bool FULL, bool ACCUMULATE>
__global__ __launch_bounds__(256) void blocked_ell_f32(const int32_t *__restrict__ ell_col, const float *__restrict__ ell_val,
                                                       uint32_t block_size, uint32_t width, uint32_t num_strips,
                                                       uint32_t num_rows, const float *__restrict__ B, float *__restrict__ C,
                                                       uint32_t N)
{
    typedef typename Vec<VEC>::type V;
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    // neighbouring strips reference neighbouring block columns: keep them on one XCD, whose L2 then holds
    // their B rows (gridDim.x is a multiple of the XCD count)
    const uint32_t strip = xcd_contiguous_id(blockIdx.x, gridDim.x / kNumXcd) * (blockDim.x / kWaveSize) +
                           __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    if (strip >= num_strips) return;
    const uint32_t row16 = lane & 15u, q = lane >> 4;
    const uint32_t c0 = blockIdx.y * (16u * VEC) + row16 * VEC;       // this lane's VEC columns of the slab
    const bool col_live = FULL || c0 < N;
    const uint32_t block_row = (strip * 16u) / block_size;
    const uint32_t tiles_per_block = block_size / 16u;                // 16-wide k tiles of one block
    const size_t pitch = size_t(width) * block_size;
    const float *a_row = ell_val + size_t(strip * 16u + row16) * pitch + q * 4u;
    const int32_t *cols = ell_col + size_t(block_row) * width;
    const float *b_base = B + size_t(q * 4u) * N + (col_live ? c0 : 0u);

    f32x4 acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = f32x4(0.0f);

    struct Operands {
        f32x4 a;
        V b[4];
        bool past;                    // wave-uniform: the set holds a re-read of the last tile and must not count
    };
    // Block ids are taken 64 at a time into one vector register (lane i holds block w0 + i);
    // the padding (-1) that follows the last block ends the row.  Inside such a batch the k
    // tiles roll through kEllDepth operand sets: a set is refilled with tile t+kEllDepth right
    // after the MFMAs of tile t, and the id of a tile's block comes out of the register by readlane, so no load
    // depends on another load.
    for (uint32_t w0 = 0; w0 < width; w0 += kWaveSize) {
        const uint32_t in_batch = min(width - w0, uint32_t(kWaveSize));
        const int32_t ids = lane < in_batch ? cols[w0 + lane] : -1;
        const uint64_t pad = __ballot(ids < 0);
        const uint32_t valid = pad ? uint32_t(__builtin_ctzll(pad)) : uint32_t(kWaveSize);
        const uint32_t tiles = valid * tiles_per_block;
        if (tiles == 0) break;
        auto fetch = [&](uint32_t t, Operands &o) {
            o.past = t >= tiles;                                      // past the end: re-read the last tile
            t = min(t, tiles - 1u);
            const uint32_t w = t / tiles_per_block, kt = (t % tiles_per_block) * 16u;
            const uint32_t bc = uint32_t(__builtin_amdgcn_readlane(ids, w));
            o.a = *reinterpret_cast<const f32x4 *>(a_row + size_t(w0 + w) * block_size + kt);
            const float *b_row = b_base + size_t(bc * block_size + kt) * N;
#pragma unroll
            for (int e = 0; e < 4; ++e) o.b[e] = *reinterpret_cast<const V *>(b_row + size_t(e) * N);
        };
        auto multiply = [&](const Operands &o) {
            const f32x4 a = o.past ? f32x4(0.0f) : o.a;               // masked here, where the data is waited for anyway
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int v = 0; v < VEC; ++v)
                    acc[v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], vec_get<VEC>(o.b[e], v), acc[v], 0, 0, 0);
        };
        Operands o[kEllDepth];
#pragma unroll
        for (int k = 0; k < kEllDepth; ++k) fetch(uint32_t(k), o[k]);
        __builtin_amdgcn_sched_barrier(0);
        for (uint32_t t = 0; t < tiles; t += kEllDepth) {
#pragma unroll
            for (int k = 0; k < kEllDepth; ++k) {
                // the fences keep the compiler from sinking the loads to their first use
                multiply(o[k]);
                __builtin_amdgcn_sched_barrier(0);
                fetch(t + uint32_t(k) + kEllDepth, o[k]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (valid < in_batch) break;
    }
    if (!col_live) return;
    const uint32_t r0 = strip * 16u + q * 4u;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (r0 + r >= num_rows) break;
        V *dst = reinterpret_cast<V *>(C + size_t(r0 + r) * N + c0);
        V out;
#pragma unroll
        for (int v = 0; v < VEC; ++v) vec_set<VEC>(out, v, acc[v][r]);
        if (ACCUMULATE) out += *dst;
        *dst = out;
    }
}

// Adds up the partial tiles of the panels (16 rows) or strips (4 rows) that were cut into several chunks:
// fixups[i] = {panel or strip, first piece, number of pieces, -}; piece k is rows [k*rows, (k+1)*rows) of the
// partials matrix, whose row pitch is N like C's.  A block of sixteen wavefronts works on tile i in segments
// of 64 elements.  With few pieces every wavefront takes a segment of its own; with many, G = 2..16
// wavefronts share a segment, wavefront g adding the pieces g, g+G, g+2G, ... (independent loads, four at a
// time), and their sums are then added in wavefront order.  G depends on the piece count alone and every
// order is fixed, so the result does not depend on which chunk finished first: the same product gives the
// same bits every time.  The launch has one block per (tile, segment); blocks past the last segment group exit.
constexpr int kReduceWaves = 16;

__global__ __launch_bounds__(kWaveSize *kReduceWaves) void reduce_partials(const uint4 *__restrict__ fixups, uint32_t count,
                                                                           uint32_t rows, const float *__restrict__ partials,
                                                                           float *__restrict__ C, uint32_t N)
{
    __shared__ float sums[kReduceWaves][kWaveSize];
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    if (blockIdx.x >= count) return;
    const uint4 fx = fixups[blockIdx.x];
    const uint32_t pieces = __builtin_amdgcn_readfirstlane(fx.z);
    const uint32_t G = pieces <= 4 ? 1u : pieces <= 8 ? 2u : pieces <= 16 ? 4u : pieces <= 32 ? 8u : 16u;
    const uint32_t segs_per_block = kReduceWaves / G;
    const uint32_t tile = rows * N;
    if (blockIdx.y * segs_per_block * kWaveSize >= tile) return;      // whole block: nothing left of this tile
    const uint32_t seg = blockIdx.y * segs_per_block + wave / G, g = wave % G;
    const uint32_t e = seg * kWaveSize + lane;
    const bool valid = e < tile;
    const float *src = partials + size_t(fx.y) * tile + (valid ? e : 0u);
    float sum = 0.0f;
    uint32_t k = g;
    for (; k < pieces; k += 4u * G) {          // four loads in flight; a piece past the end counts as zero
        const float p0 = src[size_t(k) * tile];
        const float p1 = k + G < pieces ? src[size_t(k + G) * tile] : 0.0f;
        const float p2 = k + 2u * G < pieces ? src[size_t(k + 2u * G) * tile] : 0.0f;
        const float p3 = k + 3u * G < pieces ? src[size_t(k + 3u * G) * tile] : 0.0f;
        sum = (((sum + p0) + p1) + p2) + p3;
    }
    if (G > 1) {
        sums[wave][lane] = sum;
        __syncthreads();
        if (g != 0) return;
        for (uint32_t w = 1; w < G; ++w) sum += sums[wave + w][lane];
    }
    if (valid) __builtin_nontemporal_store(sum, C + size_t(fx.x) * tile + e);
}

// One group of L = 1<<LOG_L lanes per row; lane t of the group owns VEC consecutive columns
// starting at slab*L*VEC + t*VEC.  Nonzeros are fetched L at a time, one per lane, then
// broadcast one after the other, so each C element accumulates its row in storage order.
// row_list == nullptr: rows 0..num_rows-1.
template <int VEC, int LOG_L>
__global__ __launch_bounds__(256) void csr_rows(const uint32_t *__restrict__ row_list, uint32_t num_rows,
                                                uint32_t num_slabs, const uint32_t *__restrict__ rowPtr,
                                                const uint32_t *__restrict__ cols, const float *__restrict__ vals,
                                                const float *__restrict__ B, float *__restrict__ C, uint32_t N)
{
    typedef typename Vec<VEC>::type V;
    constexpr uint32_t L = 1u << LOG_L;
    const uint32_t t = threadIdx.x & (L - 1);
    const uint64_t gid = (uint64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> LOG_L;
    // whole groups leave together, so shuffles below never read a retired lane of the same group
    if (gid >= uint64_t(num_rows) * num_slabs) return;
    const uint32_t ridx = uint32_t(gid / num_slabs);
    const uint32_t slab = uint32_t(gid % num_slabs);
    const uint32_t row = row_list ? row_list[ridx] : ridx;
    const uint32_t c0 = slab * L * VEC + t * VEC;
    const bool live = c0 < N;
    const uint32_t s = rowPtr[row], e = rowPtr[row + 1];
    V acc = V(0.0f);
    for (uint32_t base = s; base < e; base += L) {
        const uint32_t mine = base + t;
        uint32_t my_col = 0;
        float my_val = 0.0f;
        if (mine < e) { my_col = cols[mine]; my_val = vals[mine]; }
        const uint32_t cnt = min(L, e - base);
        for (uint32_t q = 0; q < cnt; ++q) {
            const uint32_t c = __shfl(my_col, int(q), int(L));
            const float a = __shfl(my_val, int(q), int(L));
            if (live) {
                const V b = *reinterpret_cast<const V *>(B + size_t(c) * N + c0);
                acc += a * b;
            }
        }
    }
    if (live) *reinterpret_cast<V *>(C + size_t(row) * N + c0) = acc;
}

// The sparse-panel kernel of the library: same work split as csr_rows, but the nonzeros of a
// row are consumed in batches whose B-row loads are all issued before the first FMA, so a
// row costs about one memory round trip per batch instead of one per nonzero.  Each C
// element still accumulates its row in storage order.
template <int VEC, int LOG_L, int BATCH>
__device__ __forceinline__ void rows_batched_body(uint32_t block_id, uint32_t slab, const uint4 *__restrict__ row_list,
                                                  uint32_t num_rows, const uint32_t *__restrict__ rowPtr,
                                                  const uint32_t *__restrict__ cols, const float *__restrict__ vals,
                                                  const float *__restrict__ B, float *__restrict__ C, uint32_t N)
{
    typedef typename Vec<VEC>::type V;
    constexpr uint32_t L = 1u << LOG_L;
    constexpr uint32_t STEP = BATCH < int(L) ? uint32_t(BATCH) : L;
    const uint32_t t = threadIdx.x & (L - 1);
    const uint64_t gid = (uint64_t(block_id) * blockDim.x + threadIdx.x) >> LOG_L;
    if (gid >= num_rows) return;
    const uint32_t ridx = uint32_t(gid);
    // a listed row comes with its row pointers {row, first entry, end, -}: one fetch, where the row index in one array
    // and the row pointers in another would be two, the second waiting for the first
    uint32_t row, s, e;
    if (row_list) {
        const uint4 entry = row_list[ridx];
        row = entry.x; s = entry.y; e = entry.z;
    } else {
        row = ridx; s = rowPtr[row]; e = rowPtr[row + 1];
    }
    const uint32_t c0 = slab * L * VEC + t * VEC;
    const bool live = c0 < N;
    const float *bcol = B + c0;
    V acc = V(0.0f);
    for (uint32_t base = s; base < e; base += L) {
        const uint32_t mine = base + t;
        uint32_t my_col = 0;
        float my_val = 0.0f;
        if (mine < e) { my_col = cols[mine]; my_val = vals[mine]; }
        const uint32_t cnt = min(L, e - base);
        for (uint32_t q0 = 0; q0 < cnt; q0 += STEP) {
            V b[STEP];
            float a[STEP];
#pragma unroll
            for (uint32_t u = 0; u < STEP; ++u) {
                // lanes past the end of the row hold (col 0, val 0): their slot is skipped
                const uint32_t c = __shfl(my_col, int(q0 + u), int(L));
                a[u] = __shfl(my_val, int(q0 + u), int(L));
                b[u] = V(0.0f);
                if (live && q0 + u < cnt) b[u] = *reinterpret_cast<const V *>(bcol + size_t(c) * N);
            }
#pragma unroll
            for (uint32_t u = 0; u < STEP; ++u) acc += a[u] * b[u];
        }
    }
    if (live) __builtin_nontemporal_store(acc, reinterpret_cast<V *>(C + size_t(row) * N + c0));
}

template <int VEC, int LOG_L, int BATCH>
__global__ __launch_bounds__(256) void csr_rows_batched(const uint4 *__restrict__ row_list, uint32_t num_rows,
                                                        const uint32_t *__restrict__ rowPtr,
                                                        const uint32_t *__restrict__ cols,
                                                        const float *__restrict__ vals, const float *__restrict__ B,
                                                        float *__restrict__ C, uint32_t N, XcdRanges ranges)
{
    // each XCD walks one contiguous range of rows (ranges of equal work), so the B rows that neighbouring
    // rows share stay in that XCD's L2.  A product wider than one lane group's slab (2^LOG_L * VEC columns) is
    // walked slab by slab, each over all rows (y is the slower index of the order in which work-groups start):
    // what the resident rows read of B at one time is then one slab wide, whatever N is.
    uint32_t block_id;
    if (!xcd_range_id(ranges, blockIdx.x, block_id)) return;
    rows_batched_body<VEC, LOG_L, BATCH>(block_id, blockIdx.y, row_list, num_rows, rowPtr, cols, vals, B, C, N);
}

// One launch for a plan that uses both the quad kernel and the row kernel: they write disjoint
// panels, and the row kernel's short, even work fills the SIMDs that the quad kernel's long chunks
// leave idle.  Blocks [0, quad_blocks) are the quad kernel's 2-D grid flattened (x fastest, so the
// XCD of a block is still x % 8); the rest are the row kernel's blocks, dealt to the XCDs in
// contiguous ranges like the row kernel's own launch does.
template <bool FULL, bool STRIPS, int LOG_L>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup, 8) void hrpb_quad_rows_f32(
    uint32_t quad_blocks_x, uint32_t quad_blocks, const uint32_t *__restrict__ heads, uint32_t num_chunks,
    uint32_t groups_per_xcd, const uint32_t *__restrict__ qrecs, const float *__restrict__ qvals, uint32_t zero_index,
    const uint4 *__restrict__ row_list, uint32_t num_rows, uint32_t row_blocks_per_slab, XcdRanges row_ranges,
    const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols, const float *__restrict__ vals,
    const float *__restrict__ B, float *__restrict__ C, float *__restrict__ partials, uint32_t N)
{
    static_assert(kWaveSize * kWavesPerGroup == 256, "both bodies are written for 256-thread blocks");
    if (blockIdx.x < quad_blocks) {
        quad_body<FULL, STRIPS>(blockIdx.x % quad_blocks_x, blockIdx.x / quad_blocks_x, heads, num_chunks, groups_per_xcd,
                                qrecs, qvals, zero_index, B, C, partials, N);
    } else {   // quad_blocks is a multiple of the XCD count, so the XCD of a row block is (its index) % 8 as well
        const uint32_t rb = blockIdx.x - quad_blocks, slab = rb / row_blocks_per_slab;      // slab by slab, as in csr_rows_batched
        uint32_t block_id;
        if (!xcd_range_id(row_ranges, rb - slab * row_blocks_per_slab, block_id)) return;
        rows_batched_body<4, LOG_L, 8>(block_id, slab, row_list, num_rows, rowPtr, cols, vals, B, C, N);
    }
}

// The same for a plan that pairs the rolling brick kernel with the row kernel.
template <int VEC, int NG, bool FULL, int LOG_L>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup, (NG == 1 ? 8 : 4)) void hrpb_brick_rows_f32(
    uint32_t brick_blocks_x, uint32_t brick_blocks, const uint4 *__restrict__ chunks, uint32_t num_chunks,
    uint32_t groups_per_xcd, const uint32_t *__restrict__ hdr, const float *__restrict__ tile_vals, uint32_t zero_index,
    const uint4 *__restrict__ row_list, uint32_t num_rows, uint32_t row_blocks_per_slab, XcdRanges row_ranges,
    const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols, const float *__restrict__ vals,
    const float *__restrict__ B, float *__restrict__ C, float *__restrict__ partials, uint32_t N)
{
    if (blockIdx.x < brick_blocks) {
        brick_rolling_body<VEC, NG, FULL>(blockIdx.x % brick_blocks_x, blockIdx.x / brick_blocks_x, chunks, num_chunks,
                                          groups_per_xcd, hdr, tile_vals, zero_index, B, C, partials, N);
    } else {
        const uint32_t rb = blockIdx.x - brick_blocks, slab = rb / row_blocks_per_slab;
        uint32_t block_id;
        if (!xcd_range_id(row_ranges, rb - slab * row_blocks_per_slab, block_id)) return;
        rows_batched_body<4, LOG_L, 8>(block_id, slab, row_list, num_rows, rowPtr, cols, vals, B, C, N);
    }
}

// Thread per C element (inc/SPMM.cuh:898-920 restated for fp32 and a 64x4 thread tile).
__global__ __launch_bounds__(256) void csr_thread_per_element(const uint32_t *__restrict__ rowPtr,
                                                              const uint32_t *__restrict__ cols,
                                                              const float *__restrict__ vals,
                                                              const float *__restrict__ B, float *__restrict__ C,
                                                              uint32_t M, uint32_t N)
{
    const uint32_t col = blockIdx.x * 64u + threadIdx.x;
    const uint32_t row = blockIdx.y * 4u + threadIdx.y;
    if (row >= M || col >= N) return;
    float sum = 0.0f;
    for (uint32_t i = rowPtr[row]; i < rowPtr[row + 1]; ++i) sum += vals[i] * B[size_t(cols[i]) * N + col];
    C[size_t(row) * N + col] = sum;
}

// Wavefront per row, lane L handles columns L, L+64, ...; every lane reads (col, val) itself.
__global__ __launch_bounds__(256) void csr_wave_scalar(const uint32_t *__restrict__ rowPtr,
                                                       const uint32_t *__restrict__ cols,
                                                       const float *__restrict__ vals, const float *__restrict__ B,
                                                       float *__restrict__ C, uint32_t M, uint32_t N)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t row = (uint64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
    if (row >= M) return;
    const uint32_t s = rowPtr[row], e = rowPtr[row + 1];
    for (uint32_t c = lane; c < N; c += 64u) {
        float sum = 0.0f;
        for (uint32_t i = s; i < e; ++i) sum += vals[i] * B[size_t(cols[i]) * N + c];
        C[row * N + c] = sum;
    }
}

}  // namespace cute_dev
