// gfx950 kernels that build the two MFMA layouts (brick tiles, quad lists) from a CSR matrix that already
// lives on the device -- the device-side counterpart of HRPB::DATASTRUCT (reference data.cu:94-335), whose
// output the host functions cute_hrpb_build + cute_hrpb_retile and cute_quad_census + cute_quad_pack
// define word for word.
//
// Both layouts are orderings of the matrix entries: the brick tiles hold the entries of a 16-row panel
// sorted by (column, row) -- active column a of the panel is column a%4 of brick (a%16)/4 of block a/16, and
// inside a brick the lane-order bitmap runs column-major -- and the quad lists hold the entries of a 4-row
// strip in the same order.  Rows are sorted and duplicate-free (checked first), so an entry finds its place
// without any sort: its position is the number of entries of its panel (strip) with a smaller column, which
// is a sum of binary searches over the panel's 16 rows, plus the rows above it that hold the same column.
// An entry is the first of its column when no row above it holds that column; a prefix sum over these
// flags, taken in sorted order, numbers the active columns.  Everything else is a scatter.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cutespmm.h"

namespace cute_build {

constexpr int kThreads = 256;
constexpr int kScanItems = 8;                               // entries per thread of a scan block
constexpr uint32_t kScanBlock = kThreads * kScanItems;      // entries per scan block

enum : int { kErrRange = 1, kErrUnsorted = 2 };

__device__ __forceinline__ uint64_t global_id() { return uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; }

// ------------------------------------------------------------------------------------------------
// Inclusive prefix sum of uint32 values, in three steps: block sums, their prefix sum (by the same three
// steps), block-local prefix sums shifted by the sums of the blocks before.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void scan_block_sums(const uint32_t *__restrict__ in, uint64_t n, uint32_t *__restrict__ sums)
{
    __shared__ uint32_t wave_sum[kThreads / 64];
    const uint64_t base = uint64_t(blockIdx.x) * kScanBlock + uint64_t(threadIdx.x) * kScanItems;
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i)
        if (base + i < n) s += in[base + i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off, 64);
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
#pragma unroll
        for (int w = 0; w < kThreads / 64; ++w) t += wave_sum[w];
        sums[blockIdx.x] = t;
    }
}

// `sums` holds the inclusive prefix sums of the block sums (nullptr when there is one block); in == out is allowed.
__global__ __launch_bounds__(kThreads) void scan_block_apply(const uint32_t *in, uint32_t *out, uint64_t n, const uint32_t *__restrict__ sums)
{
    __shared__ uint32_t wave_total[kThreads / 64];
    const uint64_t base = uint64_t(blockIdx.x) * kScanBlock + uint64_t(threadIdx.x) * kScanItems;
    uint32_t v[kScanItems];
    uint32_t t = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
        t += base + i < n ? in[base + i] : 0u;
        v[i] = t;
    }
    uint32_t incl = t;                                       // inclusive sum over the lanes of this wavefront
    const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off, 64);
        if (lane >= uint32_t(off)) incl += up;
    }
    if (lane == 63u) wave_total[threadIdx.x >> 6] = incl;
    __syncthreads();
    uint32_t offset = (sums && blockIdx.x) ? sums[blockIdx.x - 1] : 0u;
    for (uint32_t w = 0; w < (threadIdx.x >> 6); ++w) offset += wave_total[w];
    offset += incl - t;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i)
        if (base + i < n) out[base + i] = offset + v[i];
}

// ------------------------------------------------------------------------------------------------
// Entry -> row, and the preconditions of the format (data.cu:204,256-258 relies on them; here they are
// checked): every column below K, strictly increasing inside a row.  rowPtr has been checked on the host.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void row_of_entries(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols,
                                                           uint32_t M, uint32_t K, uint32_t nnz, uint32_t *__restrict__ rowOf,
                                                           int *__restrict__ error)
{
    const uint64_t e = global_id();
    if (e >= nnz) return;
    uint32_t lo = 0, hi = M - 1u;                            // the row r with rowPtr[r] <= e < rowPtr[r+1]
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (rowPtr[mid + 1] <= e) lo = mid + 1u;
        else hi = mid;
    }
    rowOf[e] = lo;
    const uint32_t c = cols[e];
    if (c >= K) atomicOr(error, int(kErrRange));
    if (e > rowPtr[lo] && cols[e - 1] >= c) atomicOr(error, int(kErrUnsorted));
}

__device__ __forceinline__ uint32_t lower_bound(const uint32_t *__restrict__ cols, uint32_t lo, uint32_t hi, uint32_t c)
{
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (cols[mid] < c) lo = mid + 1u;
        else hi = mid;
    }
    return lo;
}

// Position of every entry in the (column, row) order of its 16-row panel (posP) and of its 4-row strip (posS),
// and, at those positions, whether the entry is the first of its column there (firstP, firstS).
__global__ __launch_bounds__(kThreads) void entry_positions(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols,
                                                            const uint32_t *__restrict__ rowOf, uint32_t nnz,
                                                            uint32_t *__restrict__ posP, uint32_t *__restrict__ posS,
                                                            uint32_t *__restrict__ firstP, uint32_t *__restrict__ firstS)
{
    const uint64_t e = global_id();
    if (e >= nnz) return;
    const uint32_t r = rowOf[e], c = cols[e];
    const uint32_t r0 = r & ~15u, me = r - r0, strip0 = me & ~3u;
    uint32_t below = 0, above_same = 0, below_s = 0, above_same_s = 0;
    uint32_t lo = rowPtr[r0];
    const uint32_t panel_start = lo;
    uint32_t strip_start = 0;
    for (uint32_t i = 0; i < 16u; ++i) {
        const uint32_t hi = rowPtr[r0 + i + 1u];
        if (i == strip0) strip_start = lo;
        uint32_t cnt, has = 0;
        if (i == me) cnt = uint32_t(e) - lo;
        else {
            const uint32_t lb = lower_bound(cols, lo, hi, c);
            cnt = lb - lo;
            has = (lb < hi && cols[lb] == c) ? 1u : 0u;
        }
        below += cnt;
        if (i < me) above_same += has;
        if ((i & ~3u) == strip0) {
            below_s += cnt;
            if (i < me) above_same_s += has;
        }
        lo = hi;
    }
    const uint32_t pp = panel_start + below + above_same, ps = strip_start + below_s + above_same_s;
    posP[e] = pp;
    posS[e] = ps;
    firstP[pp] = above_same == 0u ? 1u : 0u;
    firstS[ps] = above_same_s == 0u ? 1u : 0u;
}

// Active columns per panel and list pairs per strip, from the prefix sums DP, DS of the first-of-column flags.
// Also the width of every panel's column window (last column - first column + 1; rows are sorted).
__global__ __launch_bounds__(kThreads) void count_columns(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols,
                                                          const uint32_t *__restrict__ DP, const uint32_t *__restrict__ DS,
                                                          uint32_t P, uint32_t *__restrict__ panelCols,
                                                          uint32_t *__restrict__ stripPairs, uint32_t *__restrict__ panelSpan)
{
    const uint64_t id = global_id();
    if (id < P) {
        const uint32_t s = rowPtr[id * 16u], e = rowPtr[id * 16u + 16u];
        panelCols[id] = e > s ? DP[e - 1u] - DP[s] + 1u : 0u;
        uint32_t lo = ~0u, hi = 0u;
        for (uint32_t r = 0; r < 16u; ++r) {
            const uint32_t rs = rowPtr[id * 16u + r], re = rowPtr[id * 16u + r + 1u];
            if (re > rs) { lo = min(lo, cols[rs]); hi = max(hi, cols[re - 1u]); }
        }
        panelSpan[id] = e > s ? hi - lo + 1u : 0u;
    }
    if (id < uint64_t(P) * 4u) {
        const uint32_t s = rowPtr[id * 4u], e = rowPtr[id * 4u + 4u];
        stripPairs[id] = e > s ? DS[e - 1u] - DS[s] + 1u : 0u;
    }
}

// ------------------------------------------------------------------------------------------------
// Brick tiles: hdr[nb][32] (zeroed before) and vals[] in (panel, column, row) order.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void brick_scatter(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols,
                                                          const float *__restrict__ vals, const uint32_t *__restrict__ rowOf,
                                                          const uint32_t *__restrict__ posP, const uint32_t *__restrict__ DP,
                                                          const uint32_t *__restrict__ brp, uint32_t nnz, uint32_t *hdr,
                                                          float *__restrict__ tile_vals)
{
    const uint64_t e = global_id();
    if (e >= nnz) return;
    const uint32_t r = rowOf[e], p = r >> 4, row = r & 15u, pos = posP[e], start = rowPtr[p << 4];
    const uint32_t a = DP[pos] - DP[start];                  // index of the entry's column among the panel's active columns
    const uint32_t j = (a >> 2) & 3u, k = a & 3u;
    uint32_t *h = hdr + (size_t(brp[p]) + (a >> 4)) * CUTE_TILED_HDR_WORDS;
    tile_vals[pos] = vals[e];
    const uint32_t bit = k * 16u + row;                      // the A operand slot of lane `bit` in v_mfma_f32_16x16x4_f32
    atomicOr(h + 16u + 2u * j + (bit >> 5), 1u << (bit & 31u));
    if (pos == start || DP[pos] != DP[pos - 1u]) {           // first entry of its column: the column's own words
        h[k * 4u + j] = cols[e];
        if (k == 0u) h[24u + j] = pos;
    }
}

// Per block: value offsets of bricks that hold padding columns only (they point at the end of the block, where
// a running offset would stand) and the number of entries in the block.
__global__ __launch_bounds__(kThreads) void brick_finish(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ brp,
                                                         const uint32_t *__restrict__ panelCols, uint32_t P, uint32_t nb, uint32_t *hdr)
{
    const uint64_t b = global_id();
    if (b >= nb) return;
    uint32_t lo = 0, hi = P - 1u;                            // the panel p with brp[p] <= b < brp[p+1]
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (brp[mid + 1] <= b) lo = mid + 1u;
        else hi = mid;
    }
    const uint32_t p = lo;
    uint32_t *h = hdr + size_t(b) * CUTE_TILED_HDR_WORDS;
    const uint32_t end = (b + 1u == brp[p + 1u]) ? rowPtr[p * 16u + 16u] : hdr[size_t(b + 1u) * CUTE_TILED_HDR_WORDS + 24u];
    const uint32_t live = min(16u, panelCols[p] - 16u * (uint32_t(b) - brp[p]));
    for (uint32_t j = 1; j < 4u; ++j)
        if (4u * j >= live) h[24u + j] = end;
    h[28] = end - h[24];
}

// ------------------------------------------------------------------------------------------------
// Quad lists: recs[numGroups][20] (zeroed before) and the stored values in slot order.
// STRIPS: one list per 4-row strip (unit = strip, a group = 16 consecutive pairs); else four lockstep lists
// per panel (unit = panel, pair 4*step + list).
// ------------------------------------------------------------------------------------------------
template <bool STRIPS>
__device__ __forceinline__ void quad_place(uint32_t r, uint32_t pos, const uint32_t *__restrict__ rowPtr,
                                           const uint32_t *__restrict__ DS, const uint32_t *__restrict__ qgp, uint32_t &group,
                                           uint32_t &pair, bool &first)
{
    const uint32_t s = r >> 2, start = rowPtr[s << 2];
    const uint32_t q = DS[pos] - DS[start];                  // index of the entry's column in the strip's list
    if (STRIPS) {
        group = qgp[s] + (q >> 4);
        pair = q & 15u;
    } else {
        group = qgp[r >> 4] + (q >> 2);
        pair = 4u * (q & 3u) + (s & 3u);
    }
    first = pos == start || DS[pos] != DS[pos - 1u];
}

template <bool STRIPS>
__global__ __launch_bounds__(kThreads) void quad_scatter(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols,
                                                         const float *__restrict__ vals, const uint32_t *__restrict__ rowOf,
                                                         const uint32_t *__restrict__ posS, const uint32_t *__restrict__ DS,
                                                         const uint32_t *__restrict__ qgp, uint32_t nnz, uint32_t *recs)
{
    const uint64_t e = global_id();
    if (e >= nnz) return;
    const uint32_t r = rowOf[e];
    uint32_t g, pair;
    bool first;
    quad_place<STRIPS>(r, posS[e], rowPtr, DS, qgp, g, pair, first);
    uint32_t *rec = recs + size_t(g) * CUTE_QUAD_RECORD_WORDS;
    const uint32_t slot = 4u * pair + (r & 3u);
    if (vals[e] != 0.0f) atomicOr(rec + 16u + (slot >> 5), 1u << (slot & 31u));   // an explicit zero is an empty slot
    if (first) rec[pair] = cols[e];
}

// Per group: the number of stored values (for the prefix sum that gives each group its first value) and the
// columns of padding pairs, which repeat the last column of their list (0 for an empty list).
template <bool STRIPS>
__global__ __launch_bounds__(kThreads) void quad_groups(const uint32_t *__restrict__ rowPtr, const uint32_t *__restrict__ cols,
                                                        const uint32_t *__restrict__ qgp, uint32_t U,
                                                        const uint32_t *__restrict__ stripPairs, uint32_t numGroups, uint32_t *recs,
                                                        uint32_t *__restrict__ counts)
{
    const uint64_t g = global_id();
    if (g >= numGroups) return;
    uint32_t lo = 0, hi = U - 1u;                            // the unit u with qgp[u] <= g < qgp[u+1]
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (qgp[mid + 1] <= g) lo = mid + 1u;
        else hi = mid;
    }
    const uint32_t u = lo, local = uint32_t(g) - qgp[u];
    uint32_t *rec = recs + size_t(g) * CUTE_QUAD_RECORD_WORDS;
    counts[g] = uint32_t(__popc(rec[16]) + __popc(rec[17]));
    const uint32_t lists = STRIPS ? 1u : 4u;
    for (uint32_t l = 0; l < lists; ++l) {
        const uint32_t strip = STRIPS ? u : 4u * u + l;
        const uint32_t len = stripPairs[strip];
        // steps of this list inside the group: 16 (strips) or 4 (lockstep)
        const uint32_t per = STRIPS ? 16u : 4u, first_step = local * per;
        if (first_step + per <= len) continue;               // no padding in this list here
        uint32_t last = 0;
        if (len)
            for (uint32_t i = 0; i < 4u; ++i) {
                const uint32_t s = rowPtr[strip * 4u + i], e = rowPtr[strip * 4u + i + 1u];
                if (e > s) last = max(last, cols[e - 1u]);
            }
        for (uint32_t t = 0; t < per; ++t)
            if (first_step + t >= len) rec[STRIPS ? t : 4u * t + l] = last;
    }
}

// counts holds the inclusive prefix sums of the stored values per group: word 18 of a record is the index of
// the group's first stored value.
__global__ __launch_bounds__(kThreads) void quad_first_values(const uint32_t *__restrict__ counts, uint32_t numGroups, uint32_t *recs)
{
    const uint64_t g = global_id();
    if (g >= numGroups) return;
    recs[size_t(g) * CUTE_QUAD_RECORD_WORDS + 18u] = g ? counts[g - 1u] : 0u;
}

template <bool STRIPS>
__global__ __launch_bounds__(kThreads) void quad_values(const uint32_t *__restrict__ rowPtr, const float *__restrict__ vals,
                                                        const uint32_t *__restrict__ rowOf, const uint32_t *__restrict__ posS,
                                                        const uint32_t *__restrict__ DS, const uint32_t *__restrict__ qgp,
                                                        uint32_t nnz, const uint32_t *__restrict__ recs, float *__restrict__ packed)
{
    const uint64_t e = global_id();
    if (e >= nnz) return;
    const float v = vals[e];
    if (v == 0.0f) return;
    const uint32_t r = rowOf[e];
    uint32_t g, pair;
    bool first;
    quad_place<STRIPS>(r, posS[e], rowPtr, DS, qgp, g, pair, first);
    const uint32_t *rec = recs + size_t(g) * CUTE_QUAD_RECORD_WORDS;
    const uint32_t slot = 4u * pair + (r & 3u);
    const uint64_t mask = (uint64_t(rec[17]) << 32) | rec[16];
    const uint32_t rank = uint32_t(__popcll(mask & ((1ull << slot) - 1ull)));
    packed[rec[18] + rank] = v;
}

// One 128-byte head per work item of a quad plan: its descriptor and a copy of its first group's record.
__global__ __launch_bounds__(kThreads) void quad_heads(const uint4 *__restrict__ chunks, uint32_t numChunks,
                                                       const uint32_t *__restrict__ recs, uint32_t head_words, uint32_t *__restrict__ heads)
{
    const uint64_t id = global_id();
    const uint64_t i = id / head_words;
    const uint32_t w = uint32_t(id % head_words);
    if (i >= numChunks) return;
    const uint4 ck = chunks[i];
    uint32_t v = 0;
    if (w == 0) v = ck.x;
    else if (w == 1) v = ck.y;
    else if (w == 2) v = ck.z;
    else if (w == 3) v = ck.w;
    else if (w < 4u + CUTE_QUAD_RECORD_WORDS && ck.x < ck.y) v = recs[size_t(ck.x) * CUTE_QUAD_RECORD_WORDS + (w - 4u)];
    heads[id] = v;
}

// The row kernel's list of a mixed plan: every listed row with its row pointers, {row, first entry, end, 0}.
__global__ __launch_bounds__(kThreads) void pack_row_list(const uint32_t *__restrict__ rows, uint32_t numRows,
                                                          const uint32_t *__restrict__ rowPtr, uint4 *__restrict__ out)
{
    const uint64_t i = global_id();
    if (i >= numRows) return;
    const uint32_t r = rows[i];
    out[i] = make_uint4(r, rowPtr[r], rowPtr[r + 1u], 0u);
}

// Hub plans (hrpb_quad_hub_f32): how often every column occurs in the quad records, and a copy of the records in
// which the columns that have a slot in the LDS table of hub rows (slot_of[col] != ~0u) name that slot instead.
__global__ __launch_bounds__(kThreads) void count_record_columns(const uint32_t *__restrict__ recs, uint64_t numGroups,
                                                                 uint32_t *__restrict__ counts)
{
    const uint64_t id = global_id();
    if (id >= numGroups * 16u) return;
    atomicAdd(&counts[recs[(id >> 4) * CUTE_QUAD_RECORD_WORDS + (id & 15u)]], 1u);
}

__global__ __launch_bounds__(kThreads) void mark_hub_columns(const uint32_t *__restrict__ recs, uint64_t numGroups,
                                                             const uint32_t *__restrict__ slot_of, uint32_t hub_flag,
                                                             uint32_t *__restrict__ out)
{
    const uint64_t id = global_id();
    if (id >= numGroups * CUTE_QUAD_RECORD_WORDS) return;
    uint32_t w = recs[id];
    if (id % CUTE_QUAD_RECORD_WORDS < 16u) {
        const uint32_t slot = slot_of[w];
        if (slot != ~0u) w = hub_flag | slot;
    }
    out[id] = w;
}

}  // namespace cute_build
