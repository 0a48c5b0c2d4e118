// Quad lists: the device layout of the 4x4x1 MFMA kernel.
//
// The canonical HRPB format (reference data.cu:97-246) groups the active columns of a 16-row
// panel into 16x4 bricks, which fit a 16-row matrix instruction.  On gfx950 the fp32 matrix
// instructions all run at the same rate and share the SIMD's issue stream with vector work, so
// what counts is how many of them a panel needs.  v_mfma_f32_4x4x1_16B_f32 with an A broadcast
// multiplies ONE column of FOUR rows into 64 output columns, so a panel only pays for the
// (4-row group, column) pairs that hold a nonzero: each of the four row groups of a panel gets
// its own sorted list of active columns, the four lists advance in lockstep (padded to the
// longest), and 16 pairs -- four steps of the four groups -- form one "group" of the layout:
//   cols[g*16 + 4*s + rg]          column of row group rg at step s of group g
//   vals[g*64 + 4*(4*s + rg) + i]  value of row 4*rg+i in that column (0 if absent)
// vals is exactly the A register of the kernel: lane 4*p+i, pair p = 4*s+rg.
#include "common.hpp"
#include "../../include/cutespmm.h"

#include <algorithm>
#include <cstring>
#include <vector>

namespace {

// Walks the merged, duplicate-free column list of rows [r0, r0+4) of a CSR matrix.  emit(col, v)
// receives each column once with the four row values (0 where a row has no entry there).
template <class Emit>
uint32_t merge_row_group(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t r0, Emit emit)
{
    uint32_t cur[4], end[4];
    for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t r = r0 + i;
        cur[i] = r < M ? rowPtr[r] : 0;
        end[i] = r < M ? rowPtr[r + 1] : 0;
    }
    uint32_t count = 0;
    for (;;) {
        uint32_t col = UINT32_MAX;
        bool any = false;
        for (uint32_t i = 0; i < 4; ++i)
            if (cur[i] < end[i]) { col = std::min(col, cols[cur[i]]); any = true; }
        if (!any) break;
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t i = 0; i < 4; ++i)
            // a duplicated (row, column) entry keeps its last value, as a dense scatter would
            while (cur[i] < end[i] && cols[cur[i]] == col) v[i] = vals[cur[i]++];
        emit(col, v);
        ++count;
    }
    return count;
}

}  // namespace

extern "C" {

void cute_quad_release(cute_quad_lists *q)
{
    if (!q) return;
    std::free(q->groupPtr);
    std::free(q->cols);
    std::free(q->vals);
    std::free(q->tail);
    std::memset(q, 0, sizeof(*q));
}

int cute_quad_fill(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, uint64_t *numGroups, uint64_t *numPairs)
{
    if (!rowPtr || !numGroups || !numPairs || (rowPtr[M] && !cols)) return CUTE_ERR_ARG;
    const uint32_t P = (M + CUTE_TM - 1) / CUTE_TM;
    std::vector<uint64_t> groups_of(P, 0), pairs_of(P, 0);
    cute::parallel_ranges(P, 64, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t q = b; q < e; ++q) {
            uint32_t longest = 0;
            for (uint32_t rg = 0; rg < 4; ++rg) {
                // values are not looked at: any non-null array of the right length does
                const uint32_t len = merge_row_group(M, rowPtr, cols, reinterpret_cast<const float *>(cols),
                                                     uint32_t(q) * CUTE_TM + rg * 4, [](uint32_t, const float *) {});
                longest = std::max(longest, len);
                pairs_of[q] += len;
            }
            groups_of[q] = (longest + 3) / 4;
        }
    });
    *numGroups = *numPairs = 0;
    for (uint32_t q = 0; q < P; ++q) { *numGroups += groups_of[q]; *numPairs += pairs_of[q]; }
    return CUTE_OK;
}

int cute_quad_build(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols, const float *vals,
                    cute_quad_lists *out)
{
    if (!out || !rowPtr || (rowPtr[M] && (!cols || !vals))) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    const uint32_t P = (M + CUTE_TM - 1) / CUTE_TM;
    out->M = M;
    out->K = K;
    out->numRowPanels = P;
    out->rowsPerList = CUTE_TM;
    out->groupPtr = cute::alloc_array<uint32_t>(uint64_t(P) + 1);
    out->tail = cute::alloc_array<uint32_t>(P);
    if (!out->groupPtr || !out->tail) { cute_quad_release(out); return CUTE_ERR_NOMEM; }
    std::vector<uint64_t> pairs_of(P, 0);

    // sweep 1: groups per panel = ceil(longest of the four lists / 4)
    cute::parallel_ranges(P, 64, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t q = b; q < e; ++q) {
            uint32_t longest = 0;
            for (uint32_t rg = 0; rg < 4; ++rg) {
                const uint32_t len = merge_row_group(M, rowPtr, cols, vals, uint32_t(q) * CUTE_TM + rg * 4,
                                                     [](uint32_t, const float *) {});
                longest = std::max(longest, len);
                pairs_of[q] += len;
            }
            out->groupPtr[q + 1] = (longest + 3) / 4;
            out->tail[q] = longest ? 4u * (longest - 4u * ((longest + 3) / 4 - 1)) : 0u;   // pair slots in use in the last group
        }
    });
    uint64_t total = 0;
    for (uint32_t q = 0; q < P; ++q) {
        total += out->groupPtr[q + 1];
        if (total > 0xffffffffull / 64) { cute_quad_release(out); return CUTE_ERR_SHAPE; }
        out->groupPtr[q + 1] = uint32_t(total);
    }
    out->numGroups = total;
    for (uint32_t q = 0; q < P; ++q) out->numPairs += pairs_of[q];
    out->cols = cute::alloc_array<uint32_t>(total * 16);
    out->vals = cute::alloc_array<float>(total * 64);     // calloc: absent entries are +0.0f
    if (!out->cols || !out->vals) { cute_quad_release(out); return CUTE_ERR_NOMEM; }

    // sweep 2: fill.  Steps past the end of a list repeat the list's last column (a B row the
    // kernel has just read) with zero values; an empty list points at column 0.
    cute::parallel_ranges(P, 64, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t q = b; q < e; ++q) {
            const uint64_t g0 = out->groupPtr[q];
            const uint32_t steps = (out->groupPtr[q + 1] - out->groupPtr[q]) * 4;
            for (uint32_t rg = 0; rg < 4; ++rg) {
                uint32_t s = 0, last = 0;
                merge_row_group(M, rowPtr, cols, vals, uint32_t(q) * CUTE_TM + rg * 4, [&](uint32_t col, const float *v) {
                    const uint64_t g = g0 + s / 4;
                    const uint32_t pair = 4 * (s % 4) + rg;
                    out->cols[g * 16 + pair] = col;
                    std::memcpy(out->vals + g * 64 + 4 * pair, v, 4 * sizeof(float));
                    last = col;
                    ++s;
                });
                for (; s < steps; ++s) out->cols[(g0 + s / 4) * 16 + 4 * (s % 4) + rg] = last;
            }
        }
    });
    return CUTE_OK;
}

// What the two layouts would hold, without building either: for every 4-row strip the length of its
// merged column list (pairs) and the number of values it stores (nonzero entries; an explicit zero in
// the input is an empty slot).  Group counts, padding and the fill of either layout follow from these.
int cute_quad_census(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t *stripPairs,
                     uint32_t *stripVals)
{
    if (!rowPtr || !stripPairs || !stripVals || (rowPtr[M] && (!cols || !vals))) return CUTE_ERR_ARG;
    const uint32_t S = (M + 3) / 4;
    cute::parallel_ranges(S, 1024, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t q = b; q < e; ++q) {
            uint32_t stored = 0;
            stripPairs[q] = merge_row_group(M, rowPtr, cols, vals, uint32_t(q) * 4, [&](uint32_t, const float *v) {
                for (int i = 0; i < 4; ++i) stored += v[i] != 0.0f;
            });
            stripVals[q] = stored;
        }
    });
    return CUTE_OK;
}

// The device form of the lists, written directly: per group a record of CUTE_QUAD_RECORD_WORDS words
// {16 columns, 64-bit mask of the occupied value slots (slot 4p+i = pair p, row i), index of the group's
// first stored value, pad} and the stored values of all groups in slot order.  rowsPerList 16: four
// lockstep lists per panel (unit = panel), 4: one list per strip (unit = strip).  groupPtr[U+1] and
// valBase[U] (index of each unit's first stored value) come from cute_quad_census; recs has
// groupPtr[U] * CUTE_QUAD_RECORD_WORDS words, packed valBase[U-1] + (values of the last unit) floats.
int cute_quad_pack(uint32_t M, const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t rowsPerList,
                   const uint32_t *groupPtr, const uint64_t *valBase, uint32_t *recs, float *packed)
{
    if (!rowPtr || !groupPtr || !valBase || !recs || !packed || (rowPtr[M] && (!cols || !vals))) return CUTE_ERR_ARG;
    if (rowsPerList != 16 && rowsPerList != 4) return CUTE_ERR_ARG;
    const uint32_t lists = rowsPerList / 4;                       // lists that advance together in one unit
    const uint32_t U = (M + rowsPerList - 1) / rowsPerList;
    cute::parallel_ranges(U, 64, [&](uint64_t b, uint64_t e, unsigned) {
        struct Pair { uint32_t col; float v[4]; };
        std::vector<Pair> list[4];
        for (uint64_t u = b; u < e; ++u) {
            for (uint32_t l = 0; l < lists; ++l) {
                list[l].clear();
                merge_row_group(M, rowPtr, cols, vals, uint32_t(u) * rowsPerList + l * 4, [&](uint32_t col, const float *v) {
                    Pair p;
                    p.col = col;
                    std::memcpy(p.v, v, sizeof(p.v));
                    list[l].push_back(p);
                });
            }
            uint64_t next_val = valBase[u];
            for (uint64_t g = groupPtr[u]; g < groupPtr[u + 1]; ++g) {
                uint32_t *rec = recs + g * CUTE_QUAD_RECORD_WORDS;
                const uint32_t local = uint32_t(g - groupPtr[u]);
                uint64_t mask = 0;
                rec[18] = uint32_t(next_val);
                rec[19] = 0;
                for (uint32_t p = 0; p < 16; ++p) {
                    // lockstep: pair p is step p/4 of list p%4; strips: pair p is entry p of the one list
                    const uint32_t l = lists == 4 ? p % 4 : 0;
                    const uint32_t step = lists == 4 ? local * 4 + p / 4 : local * 16 + p;
                    const std::vector<Pair> &src = list[l];
                    if (step < src.size()) {
                        rec[p] = src[step].col;
                        for (uint32_t i = 0; i < 4; ++i)
                            if (src[step].v[i] != 0.0f) { mask |= 1ull << (4 * p + i); packed[next_val++] = src[step].v[i]; }
                    } else {
                        rec[p] = src.empty() ? 0u : src.back().col;        // padding repeats the list's last column
                    }
                }
                rec[16] = uint32_t(mask);
                rec[17] = uint32_t(mask >> 32);
            }
        }
    });
    return CUTE_OK;
}

// The same pairs with one list per 4-row strip instead of four lockstep lists per panel: nothing
// is padded to a longer neighbour, which is what a matrix with a few very long rows needs (the
// strip holding such a row would otherwise stretch the other three of its panel).  A group is 16
// consecutive pairs of one strip: cols[g*16 + p], vals[g*64 + 4*p + i] = value of row 4*strip+i.
int cute_quad_build_strips(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols, const float *vals,
                           cute_quad_lists *out)
{
    if (!out || !rowPtr || (rowPtr[M] && (!cols || !vals))) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    const uint32_t S = (M + 3) / 4;
    out->M = M;
    out->K = K;
    out->numRowPanels = S;
    out->rowsPerList = 4;
    out->groupPtr = cute::alloc_array<uint32_t>(uint64_t(S) + 1);
    out->tail = cute::alloc_array<uint32_t>(S);
    if (!out->groupPtr || !out->tail) { cute_quad_release(out); return CUTE_ERR_NOMEM; }
    cute::parallel_ranges(S, 256, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t q = b; q < e; ++q) {
            const uint32_t len = merge_row_group(M, rowPtr, cols, vals, uint32_t(q) * 4, [](uint32_t, const float *) {});
            out->groupPtr[q + 1] = (len + 15) / 16;
            out->tail[q] = len ? len - 16u * ((len + 15) / 16 - 1) : 0u;
        }
    });
    uint64_t total = 0, pairs = 0;
    for (uint32_t q = 0; q < S; ++q) {
        const uint32_t groups = out->groupPtr[q + 1];
        pairs += groups ? uint64_t(groups - 1) * 16 + out->tail[q] : 0;
        total += groups;
        if (total > 0xffffffffull / 64) { cute_quad_release(out); return CUTE_ERR_SHAPE; }
        out->groupPtr[q + 1] = uint32_t(total);
    }
    out->numGroups = total;
    out->numPairs = pairs;
    out->cols = cute::alloc_array<uint32_t>(total * 16);
    out->vals = cute::alloc_array<float>(total * 64);
    if (!out->cols || !out->vals) { cute_quad_release(out); return CUTE_ERR_NOMEM; }
    cute::parallel_ranges(S, 256, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t q = b; q < e; ++q) {
            const uint64_t g0 = out->groupPtr[q];
            const uint32_t slots = (out->groupPtr[q + 1] - out->groupPtr[q]) * 16;
            uint32_t s = 0, last = 0;
            merge_row_group(M, rowPtr, cols, vals, uint32_t(q) * 4, [&](uint32_t col, const float *v) {
                out->cols[g0 * 16 + s] = col;
                std::memcpy(out->vals + g0 * 64 + 4 * uint64_t(s), v, 4 * sizeof(float));
                last = col;
                ++s;
            });
            for (; s < slots; ++s) out->cols[g0 * 16 + s] = last;
        }
    });
    return CUTE_OK;
}

}  // extern "C"
