// gfx950 device kernels of libcutespmm.
//
//   hrpb_brick_f32   one wavefront per (row-panel chunk, N slab); every non-empty 16x4
//                    brick is one v_mfma_f32_16x16x4_f32 A operand taken straight from the
//                    lane-order bitmap; B rows are gathered in the MFMA B-operand layout
//                    (16 lanes read one contiguous row segment) so no LDS transpose is needed.
//   csr_rows         one lane group per CSR row, lanes span N, (col, val) pairs broadcast
//                    by lane shuffles; used for sparse panels and as a plain CSR kernel.
//   csr_thread_per_element / csr_wave_scalar   the simple CSR comparison kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cute_dev {

typedef float f32x4 __attribute__((ext_vector_type(4)));
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
#ifndef CUTE_WPG
#define CUTE_WPG 4
#endif
constexpr int kWavesPerGroup = CUTE_WPG;
constexpr int kHdrWords = 32;
constexpr int kNumXcd = 8;

// Work-groups are handed to the 8 XCDs round-robin; this maps the hardware id to a
// logical id such that each XCD walks one contiguous range of logical ids (neighbouring
// row panels share B rows, which then stay in that XCD's L2).
__device__ __forceinline__ uint32_t xcd_contiguous_id(uint32_t bid, uint32_t groups_per_xcd)
{
    return (bid % kNumXcd) * groups_per_xcd + bid / kNumXcd;
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
        const float *brow = B + size_t(cols[j]) * N + col0;
#pragma unroll
        for (int ng = 0; ng < NG; ++ng) {
            if (FULL || col0 + uint32_t(ng) * 16u * VEC < N) o.b[j][ng] = *reinterpret_cast<const V *>(brow + ng * 16 * VEC);
            else o.b[j][ng] = V(0.0f);
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
#ifdef CUTE_EXPERIMENT_NO_MFMA   // timing experiment only: keeps every load alive, drops the matrix work
                acc[ng][v][0] += a * vec_get<VEC>(o.b[j][ng], v);
#else
                acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vec_get<VEC>(o.b[j][ng], v), acc[ng][v], 0, 0, 0);
#endif
    }
}

// chunks[i] = {first block, end block, row panel, atomic}.  A work item is (chunk, slab);
// slab s covers columns [s*16*VEC*NG, (s+1)*16*VEC*NG).  Lane L = 16*g + j owns, inside
// column group ng, the VEC consecutive columns starting at s*slab + ng*16*VEC + j*VEC;
// MFMA tile v of that group therefore holds the columns {.. + j*VEC + v}, and after the
// MFMA lane L holds rows 4g..4g+3 of exactly those VEC columns -> one vector store per row.
// FULL: N is a multiple of the slab width, so no column guard is compiled in.
struct BrickItem {
    uint32_t start, end, panel, atomic, col0;
    bool valid;
};

template <int VEC, int NG>
__device__ __forceinline__ BrickItem brick_item(const uint4 *__restrict__ chunks, uint32_t num_chunks,
                                                uint32_t num_slabs, uint32_t groups_per_xcd, uint32_t lane)
{
    BrickItem it;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const uint32_t group = xcd_contiguous_id(blockIdx.x, groups_per_xcd);
    const uint64_t item = uint64_t(group) * kWavesPerGroup + wave;
    it.valid = item < uint64_t(num_chunks) * num_slabs;
    if (!it.valid) return it;
    const uint32_t chunk = uint32_t(item / num_slabs);
    const uint32_t slab = uint32_t(item % num_slabs);
    const uint4 ck = chunks[chunk];
    it.start = __builtin_amdgcn_readfirstlane(ck.x);
    it.end = __builtin_amdgcn_readfirstlane(ck.y);
    it.panel = __builtin_amdgcn_readfirstlane(ck.z);
    it.atomic = __builtin_amdgcn_readfirstlane(ck.w);
    it.col0 = slab * (16u * VEC * NG) + (lane & 15u) * VEC;
    return it;
}

template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void brick_store(const BrickItem &it, const f32x4 (&acc)[NG][VEC], float *__restrict__ C,
                                            uint32_t N, uint32_t lane)
{
    typedef typename Vec<VEC>::type V;
    const uint32_t row0 = it.panel * 16u + (lane >> 4) * 4u;
#pragma unroll
    for (int ng = 0; ng < NG; ++ng) {
        const uint32_t c = it.col0 + uint32_t(ng) * 16u * VEC;
        if (!FULL && c >= N) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float *dst = C + size_t(row0 + r) * N + c;
            if (it.atomic) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) unsafeAtomicAdd(dst + v, acc[ng][v][r]);
            } else {
                V out;
#pragma unroll
                for (int v = 0; v < VEC; ++v) vec_set<VEC>(out, v, acc[ng][v][r]);
                *reinterpret_cast<V *>(dst) = out;
            }
        }
    }
}

// Variant "pipelined": two operand sets per wavefront ping-pong, so a wavefront overlaps its
// own loads with its own MFMAs.  Best when work items are long (many blocks per chunk) and
// few wavefronts fit per SIMD anyway.
template <int VEC, int NG, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup) void hrpb_brick_f32(
    const uint4 *__restrict__ chunks, uint32_t num_chunks, uint32_t num_slabs, uint32_t groups_per_xcd,
    const uint32_t *__restrict__ hdr, const float *__restrict__ vals, const float *__restrict__ B,
    float *__restrict__ C, uint32_t N)
{
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const BrickItem it = brick_item<VEC, NG>(chunks, num_chunks, num_slabs, groups_per_xcd, lane);
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
    brick_store<VEC, NG, FULL>(it, acc, C, N, lane);
}

// One brick's loads (A value at the lane's rank, B row segment(s)) -- the unit of the rolling
// pipeline below.
template <int VEC, int NG, bool FULL>
__device__ __forceinline__ void load_brick(BlockOperands<VEC, NG> &o, int j, const BlockHeader &hd,
                                           const float *__restrict__ vals, const float *__restrict__ B, uint32_t N,
                                           uint32_t col0)
{
    typedef typename Vec<VEC>::type V;
    const uint32_t cols[4] = {hd.cols.x, hd.cols.y, hd.cols.z, hd.cols.w};
    const uint64_t bm = hd.bitmap[j];
    const uint32_t below = __builtin_amdgcn_mbcnt_hi(uint32_t(bm >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(bm), 0u));
    o.a[j] = vals[hd.voff[j] + below];
    o.bitmap[j] = bm;
    const float *brow = B + size_t(cols[j]) * N + col0;
#pragma unroll
    for (int ng = 0; ng < NG; ++ng) {
        if (FULL || col0 + uint32_t(ng) * 16u * VEC < N) o.b[j][ng] = *reinterpret_cast<const V *>(brow + ng * 16 * VEC);
        else o.b[j][ng] = V(0.0f);
    }
}

template <int VEC, int NG, bool SKIP_EMPTY>
__device__ __forceinline__ void mfma_brick(const BlockOperands<VEC, NG> &o, int j, f32x4 (&acc)[NG][VEC], uint32_t lane)
{
    if (SKIP_EMPTY && o.bitmap[j] == 0) return;     // wave-uniform: a brick made of padding columns only
    const float a = ((o.bitmap[j] >> lane) & 1ull) ? o.a[j] : 0.0f;
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < VEC; ++v)
#if defined(CUTE_EXPERIMENT_NO_MFMA)
            acc[ng][v][0] += a * vec_get<VEC>(o.b[j][ng], v);
#elif defined(CUTE_EXP_MFMA_BRICKS)
            if (j < CUTE_EXP_MFMA_BRICKS) acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vec_get<VEC>(o.b[j][ng], v), acc[ng][v], 0, 0, 0);
            else acc[ng][v][0] += a * vec_get<VEC>(o.b[j][ng], v);
#else
            acc[ng][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vec_get<VEC>(o.b[j][ng], v), acc[ng][v], 0, 0, 0);
#endif
}

// Variant "rolling": ONE operand set per wavefront, refilled brick by brick -- as soon as the
// MFMAs of brick j of block i are issued, the loads of brick j of block i+1 go out into the
// same registers.  Loads are therefore always in flight behind the MFMAs, and the register
// budget (one operand set, one accumulator set) lets eight wavefronts share a SIMD, so a
// launch of short panels is resident as a whole.  Padding-only bricks skip their MFMAs.
template <int VEC, int NG, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup, 8) void hrpb_brick_f32_rolling(
    const uint4 *__restrict__ chunks, uint32_t num_chunks, uint32_t num_slabs, uint32_t groups_per_xcd,
    const uint32_t *__restrict__ hdr, const float *__restrict__ vals, const float *__restrict__ B,
    float *__restrict__ C, uint32_t N)
{
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const BrickItem it = brick_item<VEC, NG>(chunks, num_chunks, num_slabs, groups_per_xcd, lane);
    if (!it.valid) return;
    const uint32_t end = it.end, col0 = it.col0;

    f32x4 acc[NG][VEC];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[ng][v] = f32x4(0.0f);

    uint32_t blk = it.start;
    if (blk < end) {
        BlockOperands<VEC, NG> op;
        BlockHeader h1, h2;
        {
            const BlockHeader h0 = load_header(hdr, blk, lane);
            h1 = load_header(hdr, min(blk + 1, end - 1), lane);
#pragma unroll
            for (int j = 0; j < 4; ++j) load_brick<VEC, NG, FULL>(op, j, h0, vals, B, N, col0);
        }
        // One basic block per iteration and a scheduling fence after every group, so the order
        // "MFMAs of brick j, then the loads that refill brick j" survives instruction scheduling.
        // Only the last block of a panel can hold padding-only bricks; it is peeled below.
        for (; blk + 1 < end; ++blk) {       // op holds block blk, h1 the header line of blk+1
            h2 = load_header(hdr, min(blk + 2, end - 1), lane);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mfma_brick<VEC, NG, false>(op, j, acc, lane);
                __builtin_amdgcn_sched_barrier(0);
                load_brick<VEC, NG, FULL>(op, j, h1, vals, B, N, col0);
                __builtin_amdgcn_sched_barrier(0);
            }
            h1 = h2;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) mfma_brick<VEC, NG, true>(op, j, acc, lane);
    }
    brick_store<VEC, NG, FULL>(it, acc, C, N, lane);
}

// Variant "persistent": the launch holds a fixed number of wavefronts (a few per SIMD); each
// walks a contiguous run of work items, items[i] = {first block, end block, panel,
// atomic | slab << 1}.  Nothing but the first header fetch of a wavefront is exposed: header
// lines run two blocks ahead ACROSS item boundaries (the descriptors of the next two items
// are kept in scalar registers), and the store of one item overlaps the loads of the next.
// wave_items[w] .. wave_items[w+1] is the run of logical wavefront w; logical ids are laid
// out so that each XCD owns one contiguous range of items.
template <int VEC, int NG, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup) void hrpb_brick_f32_persistent(
    const uint4 *__restrict__ items, const uint32_t *__restrict__ wave_items, uint32_t waves_per_xcd,
    const uint32_t *__restrict__ hdr, const float *__restrict__ vals, const float *__restrict__ B,
    float *__restrict__ C, uint32_t N)
{
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const uint32_t logical = (blockIdx.x % kNumXcd) * waves_per_xcd + (blockIdx.x / kNumXcd) * kWavesPerGroup + wave;
    const uint32_t ib = wave_items[logical], ie = wave_items[logical + 1];
    if (ib >= ie) return;

    struct Item { uint32_t start, end, panel, flags; };
    auto fetch = [&](uint32_t i) {
        const uint4 q = items[min(i, ie - 1)];          // clamped: past the run the last item repeats
        Item r;
        r.start = __builtin_amdgcn_readfirstlane(q.x);
        r.end = __builtin_amdgcn_readfirstlane(q.y);
        r.panel = __builtin_amdgcn_readfirstlane(q.z);
        r.flags = __builtin_amdgcn_readfirstlane(q.w);
        return r;
    };
    Item cur = fetch(ib), nx1 = fetch(ib + 1), nx2 = fetch(ib + 2);
    // block id `ahead` (1 or 2) steps after block `blk` of the current item, in stream order
    auto lookahead = [&](uint32_t blk, uint32_t ahead) {
        if (blk + ahead < cur.end) return blk + ahead;
        const uint32_t over = blk + ahead - cur.end, len1 = nx1.end - nx1.start;
        return over < len1 ? nx1.start + over : nx2.start + (over - len1);
    };

    f32x4 acc[NG][VEC];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[ng][v] = f32x4(0.0f);

    // Rolling refill across item boundaries: `op` holds the current block of the stream, h1 the
    // header line of the next block of the stream (possibly the first block of the next item,
    // whose slab -- hence B column offset -- may differ), h2 the one after that.
    auto col0_of = [&](const Item &q) { return (q.flags >> 1) * (16u * VEC * NG) + (lane & 15u) * VEC; };
    BlockOperands<VEC, NG> op;
    uint32_t item = ib, blk = cur.start;
    BlockHeader h1, h2;
    {
        const BlockHeader h0 = load_header(hdr, blk, lane);
        h1 = load_header(hdr, lookahead(blk, 1), lane);
        const uint32_t c0 = col0_of(cur);
#pragma unroll
        for (int j = 0; j < 4; ++j) load_brick<VEC, NG, FULL>(op, j, h0, vals, B, N, c0);
    }
    while (true) {
        const bool last_of_item = blk + 1 == cur.end;
        const uint32_t col0_next = last_of_item ? col0_of(nx1) : col0_of(cur);
        const uint32_t blk_next = lookahead(blk, 1);
        h2 = load_header(hdr, lookahead(blk, 2), lane);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            mfma_brick<VEC, NG, false>(op, j, acc, lane);
            __builtin_amdgcn_sched_barrier(0);
            load_brick<VEC, NG, FULL>(op, j, h1, vals, B, N, col0_next);   // past the run: a harmless re-read
            __builtin_amdgcn_sched_barrier(0);
        }
        h1 = h2;
        if (last_of_item) {
            BrickItem done;
            done.panel = cur.panel;
            done.atomic = cur.flags & 1u;
            done.col0 = col0_of(cur);
            brick_store<VEC, NG, FULL>(done, acc, C, N, lane);
#pragma unroll
            for (int ng = 0; ng < NG; ++ng)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[ng][v] = f32x4(0.0f);
            if (++item == ie) break;
            cur = nx1;
            nx1 = nx2;
            nx2 = fetch(item + 2);
        }
        blk = blk_next;
    }
}

// ---------------------------------------------------------------------------------------
// Variant "stream": persistent wavefronts, each with a ring of DEPTH operand sets in registers.
//
// In the variants above every wavefront of a launch asks for its first operands at the same
// moment and writes its C tile at the same moment, so the matrix pipes idle while the first
// loads and the last stores are served.  Here a few wavefronts per SIMD each walk a long run
// of blocks: the loads of block t+DEPTH are issued as soon as the MFMAs of block t have been
// issued, C tiles are written (without waiting for them) while the following blocks are already
// in flight, and the matrix pipe starts as soon as the first block of a run has landed.
//
// The host flattens the work into one stream of blocks per wavefront:
//   step_blk[t]   block id
//   step_meta[t]  low word: row panel; high word: flags
//                 flags bit0 last step of its item (store C afterwards),
//                       bit1 combine through atomics,
//                       bit2 padding step (items are padded to a whole number of ring turns),
//                       bits 8.. slab index (64 columns per slab)
// wave_steps[w] .. wave_steps[w+1] is the run of logical wavefront w (XCD-contiguous ids); runs
// end on item boundaries.  Both step arrays are padded by DEPTH+2 repeats of the last step, so
// look-ahead never leaves them.
//
// Header lines are wave-uniform and are fetched with scalar loads only; every block issues
// exactly eight vector loads (4 A, 4 B), also past the end of a run (there the B part is pointed
// at the zero pad behind the values), so the number of loads in flight behind any operand set
// is a compile-time constant and the waits never drain the ring.
// ---------------------------------------------------------------------------------------
struct ScalarHeader {        // a whole header line in scalar registers
    uint32_t cols[16];
    uint64_t bitmap[4];
    uint32_t voff[4];
};

__device__ __forceinline__ ScalarHeader load_scalar_header(const uint32_t *__restrict__ hdr, uint32_t blk)
{
    const uint32_t *h = hdr + size_t(blk) * kHdrWords;
    ScalarHeader r;
#pragma unroll
    for (int i = 0; i < 16; ++i) r.cols[i] = h[i];
    const uint64_t *bm = reinterpret_cast<const uint64_t *>(h + 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) r.bitmap[j] = bm[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) r.voff[j] = h[24 + j];
    return r;
}

struct StreamOperands {      // one block: masked A values and B row segments of its four bricks
    float a[4];
    f32x4 b[4];
};

// keep == 0 (padding step, or a step past the end of the run) turns every A value into the stored zero.
__device__ __forceinline__ void stream_issue(StreamOperands &o, const ScalarHeader &h, const float *__restrict__ vals,
                                             uint32_t keep, uint32_t zero_index, const float *__restrict__ B, uint32_t N,
                                             uint32_t col, uint32_t lane)
{
    const uint32_t g = lane >> 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // column of lane group g in brick j: header word g*4 + j
        const uint32_t c01 = g == 0 ? h.cols[j] : h.cols[4 + j];
        const uint32_t c23 = g == 2 ? h.cols[8 + j] : h.cols[12 + j];
        const uint32_t colj = g < 2 ? c01 : c23;
        const uint64_t bm = h.bitmap[j] & (uint64_t(keep) | (uint64_t(keep) << 32));
        const uint32_t below = __builtin_amdgcn_mbcnt_hi(uint32_t(bm >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(bm), 0u));
        // lanes whose bit is clear read a stored zero, so the register holds the masked A operand
        const uint32_t aidx = ((bm >> lane) & 1ull) ? h.voff[j] + below : zero_index;
        o.a[j] = vals[aidx];
        o.b[j] = *reinterpret_cast<const f32x4 *>(B + size_t(colj) * N + col);
    }
}

template <int DEPTH, bool FULL>
__global__ __launch_bounds__(kWaveSize *kWavesPerGroup) void hrpb_brick_f32_stream(
    const uint32_t *__restrict__ step_blk, const uint64_t *__restrict__ step_meta, const uint32_t *__restrict__ wave_steps,
    uint32_t waves_per_xcd, const uint32_t *__restrict__ hdr, const float *__restrict__ vals, uint32_t zero_index,
    const float *__restrict__ B, float *__restrict__ C, uint32_t N)
{
    static_assert(DEPTH >= 2 && DEPTH <= 6, "ring depth");
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const uint32_t logical = (blockIdx.x % kNumXcd) * waves_per_xcd + (blockIdx.x / kNumXcd) * kWavesPerGroup + wave;
    const uint32_t t0 = wave_steps[logical], t1 = wave_steps[logical + 1];
    if (t0 >= t1) return;
    const uint32_t lane_col = (lane & 15u) * 4u;
    auto column_of = [&](uint32_t flags) {
        const uint32_t c = (flags >> 8) * 64u + lane_col;
        return FULL ? c : min(c, N - 4u);          // ragged tail: re-read the last full vector, masked at the store
    };
    const float *zeros = vals + zero_index;

    StreamOperands ring[DEPTH];
    // prologue: fill the ring
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) {
        const ScalarHeader h = load_scalar_header(hdr, step_blk[t0 + i]);
        const uint32_t f = uint32_t(step_meta[t0 + i] >> 32);
        const bool live = !(f & 4u);              // a run holds at least one whole item, i.e. DEPTH steps
        stream_issue(ring[i], h, vals, live ? 0xffffffffu : 0u, zero_index, live ? B : zeros, live ? N : 0u,
                     live ? column_of(f) : lane_col, lane);
    }
    // scalar look-ahead: header of step t+DEPTH (used at the end of step t), block id of t+DEPTH+1
    ScalarHeader h_issue = load_scalar_header(hdr, step_blk[t0 + DEPTH]);
    uint32_t blk_ahead = step_blk[t0 + DEPTH + 1];
    uint32_t flags_issue = uint32_t(step_meta[t0 + DEPTH] >> 32);

    uint32_t t = t0;
    do {   // one item: a whole number of ring turns that ends with a C tile
        f32x4 acc[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[v] = f32x4(0.0f);
        uint64_t meta;
        do {   // one ring turn
#pragma unroll
            for (int s = 0; s < DEPTH; ++s) {
                StreamOperands &o = ring[s];
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        acc[v] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[j], o.b[j][v], acc[v], 0, 0, 0);
                // refill the set just consumed with block t+s+DEPTH, then advance the scalar look-ahead
                {
                    const bool live = !(flags_issue & 4u) && t + s + DEPTH < t1;
                    stream_issue(o, h_issue, vals, live ? 0xffffffffu : 0u, zero_index, live ? B : zeros, live ? N : 0u,
                                 live ? column_of(flags_issue) : lane_col, lane);
                }
                h_issue = load_scalar_header(hdr, blk_ahead);
                flags_issue = uint32_t(step_meta[t + s + DEPTH + 1] >> 32);
                blk_ahead = step_blk[t + s + DEPTH + 2];
            }
            meta = step_meta[t + DEPTH - 1];
            t += DEPTH;
        } while (!(uint32_t(meta >> 32) & 1u));
        // end of the item: write its C tile; the stores are not waited for
        const uint32_t flags = uint32_t(meta >> 32);
        const uint32_t c = (flags >> 8) * 64u + lane_col;
        if (FULL || c < N) {
            const uint32_t row0 = uint32_t(meta) * 16u + (lane >> 4) * 4u;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float *dst = C + size_t(row0 + r) * N + c;
                if (flags & 2u) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) unsafeAtomicAdd(dst + v, acc[v][r]);
                } else {
                    f32x4 out;
#pragma unroll
                    for (int v = 0; v < 4; ++v) out[v] = acc[v][r];
                    *reinterpret_cast<f32x4 *>(dst) = out;
                }
            }
        }
    } while (t < t1);
}

// Zero the C rows of the listed 16-row panels (those whose chunks combine through atomics).
__global__ void zero_panels(const uint32_t *__restrict__ panels, uint32_t count, float *__restrict__ C, uint32_t N)
{
    const uint32_t p = blockIdx.x;
    if (p >= count) return;
    float *base = C + size_t(panels[p]) * 16u * N;
    for (uint32_t i = threadIdx.x; i < 16u * N; i += blockDim.x) base[i] = 0.0f;
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
__global__ __launch_bounds__(256) void csr_rows_batched(const uint32_t *__restrict__ row_list, uint32_t num_rows,
                                                        uint32_t num_slabs, const uint32_t *__restrict__ rowPtr,
                                                        const uint32_t *__restrict__ cols,
                                                        const float *__restrict__ vals, const float *__restrict__ B,
                                                        float *__restrict__ C, uint32_t N)
{
    typedef typename Vec<VEC>::type V;
    constexpr uint32_t L = 1u << LOG_L;
    constexpr uint32_t STEP = BATCH < int(L) ? uint32_t(BATCH) : L;
    const uint32_t t = threadIdx.x & (L - 1);
    const uint64_t gid = (uint64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> LOG_L;
    if (gid >= uint64_t(num_rows) * num_slabs) return;
    const uint32_t ridx = uint32_t(gid / num_slabs);
    const uint32_t slab = uint32_t(gid % num_slabs);
    const uint32_t row = row_list ? row_list[ridx] : ridx;
    const uint32_t c0 = slab * L * VEC + t * VEC;
    const bool live = c0 < N;
    const uint32_t s = rowPtr[row], e = rowPtr[row + 1];
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
    if (live) *reinterpret_cast<V *>(C + size_t(row) * N + c0) = acc;
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
