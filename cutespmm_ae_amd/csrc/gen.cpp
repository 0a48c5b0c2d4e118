// Seeded synthetic inputs: the five benchmark matrix families and dense operands.
// Every value is a pure function of (seed, stream, index), so results do not depend on
// the number of host threads or on generation order.
#include <cmath>

#include "common.hpp"

using namespace cute;

namespace {

constexpr uint64_t kPattern = 0, kValues = 1, kDense = 2;

inline float sym_unit(uint64_t h) { return 2.0f * u01(h) - 1.0f; }   // U(-1,1)

int finish(uint32_t M, uint32_t K, std::vector<uint32_t> &rowPtr, std::vector<uint32_t> &cols,
           std::vector<float> &vals, cute_csr *out)
{
    out->M = M;
    out->K = K;
    out->nnz = uint32_t(cols.size());
    out->rowPtr = alloc_array<uint32_t>(uint64_t(M) + 1);
    out->cols = alloc_array<uint32_t>(cols.size());
    out->vals = alloc_array<float>(vals.size());
    if (!out->rowPtr || !out->cols || !out->vals) { cute_csr_release(out); return CUTE_ERR_NOMEM; }
    std::memcpy(out->rowPtr, rowPtr.data(), (uint64_t(M) + 1) * sizeof(uint32_t));
    std::memcpy(out->cols, cols.data(), cols.size() * sizeof(uint32_t));
    std::memcpy(out->vals, vals.data(), vals.size() * sizeof(float));
    return CUTE_OK;
}

// `per_row` distinct columns per row drawn uniformly from [lo(r), hi(r)], sorted; U(-1,1) values.
template <class Window>
int gen_fixed_degree(uint64_t seed, uint32_t M, uint32_t per_row, Window window, cute_csr *out)
{
    if (uint64_t(M) * per_row > 0xFFFFFFFFull) return CUTE_ERR_SHAPE;
    out->M = out->K = M;
    out->nnz = M * per_row;
    out->rowPtr = alloc_array<uint32_t>(uint64_t(M) + 1);
    out->cols = alloc_array<uint32_t>(out->nnz);
    out->vals = alloc_array<float>(out->nnz);
    if (!out->rowPtr || !out->cols || !out->vals) { cute_csr_release(out); return CUTE_ERR_NOMEM; }
    int status = CUTE_OK;
    parallel_ranges(M, 1024, [&](uint64_t rb, uint64_t re, unsigned) {
        for (uint64_t r = rb; r < re; ++r) {
            uint32_t lo, hi;
            window(uint32_t(r), lo, hi);
            const uint32_t width = hi - lo + 1;
            if (width < per_row) { __atomic_store_n(&status, int(CUTE_ERR_SHAPE), __ATOMIC_RELAXED); return; }
            uint32_t *c = out->cols + r * per_row;
            uint32_t have = 0;
            for (uint64_t t = 0; have < per_row; ++t) {
                uint32_t cand = lo + uint32_t(rng_at(seed, kPattern, r * 65536ull + t) % width);
                bool dup = false;
                for (uint32_t i = 0; i < have; ++i) dup |= (c[i] == cand);
                if (!dup) c[have++] = cand;
            }
            std::sort(c, c + per_row);
            for (uint32_t i = 0; i < per_row; ++i)
                out->vals[r * per_row + i] = sym_unit(rng_at(seed, kValues, r * per_row + i));
            out->rowPtr[r + 1] = uint32_t((r + 1) * per_row);
        }
    });
    if (status != CUTE_OK) cute_csr_release(out);
    return status;
}

int gen_stencil(uint64_t seed, uint32_t g, cute_csr *out)
{
    const uint64_t M64 = uint64_t(g) * g;
    if (g < 2 || M64 * 9 > 0xFFFFFFFFull) return CUTE_ERR_SHAPE;
    const uint32_t M = uint32_t(M64);
    std::vector<uint32_t> rowPtr(uint64_t(M) + 1, 0), cols;
    std::vector<float> vals;
    cols.reserve(uint64_t(M) * 9);
    vals.reserve(uint64_t(M) * 9);
    for (uint32_t y = 0; y < g; ++y)
        for (uint32_t x = 0; x < g; ++x) {
            const uint32_t r = y * g + x;
            for (int dy = -1; dy <= 1; ++dy)
                for (int dx = -1; dx <= 1; ++dx) {
                    int yy = int(y) + dy, xx = int(x) + dx;
                    if (yy < 0 || xx < 0 || yy >= int(g) || xx >= int(g)) continue;
                    const uint32_t c = uint32_t(yy) * g + uint32_t(xx);
                    const float noise = 0.01f * sym_unit(rng_at(seed, kValues, uint64_t(r) * 16 + uint64_t((dy + 1) * 3 + dx + 1)));
                    cols.push_back(c);
                    vals.push_back((c == r ? 8.0f : -1.0f) + noise);
                }
            rowPtr[r + 1] = uint32_t(cols.size());
        }
    return finish(M, M, rowPtr, cols, vals, out);
}

int gen_fem(uint64_t seed, uint32_t nblocks, uint32_t bandwidth, cute_csr *out)
{
    constexpr uint32_t B = 6;
    if (nblocks < 2 || bandwidth < 8 || uint64_t(nblocks) * B > 0xFFFFFFF0ull) return CUTE_ERR_SHAPE;
    std::vector<std::vector<uint32_t>> adj(nblocks);
    for (uint32_t i = 0; i < nblocks; ++i) {
        adj[i].push_back(i);
        const uint32_t room = std::min(bandwidth, nblocks - 1 - i);
        const uint32_t want = std::min<uint32_t>((i & 1u) ? 4u : 5u, room);   // 4.5 upper neighbours on average
        uint32_t picked[8];
        uint32_t have = 0;
        for (uint64_t t = 0; have < want; ++t) {
            uint32_t j = i + 1 + uint32_t(rng_at(seed, kPattern, uint64_t(i) * 4096 + t) % room);
            bool dup = false;
            for (uint32_t q = 0; q < have; ++q) dup |= (picked[q] == j);
            if (dup) continue;
            picked[have++] = j;
            adj[i].push_back(j);
            adj[j].push_back(i);
        }
    }
    const uint32_t M = nblocks * B;
    std::vector<uint32_t> rowPtr(uint64_t(M) + 1, 0), cols;
    std::vector<float> vals;
    for (uint32_t i = 0; i < nblocks; ++i) {
        std::sort(adj[i].begin(), adj[i].end());
        for (uint32_t rr = 0; rr < B; ++rr) {
            const uint32_t r = i * B + rr;
            const size_t row_begin = cols.size();
            size_t diag_pos = 0;
            float offsum = 0.0f;
            for (uint32_t j : adj[i])
                for (uint32_t cc = 0; cc < B; ++cc) {
                    const uint32_t c = j * B + cc;
                    float v = sym_unit(rng_at(seed, kValues, (uint64_t(r) << 32) | c));
                    if (c == r) diag_pos = cols.size(); else offsum += std::fabs(v);
                    cols.push_back(c);
                    vals.push_back(v);
                }
            (void)row_begin;
            vals[diag_pos] = 1.0f + offsum;   // diagonally dominant
            rowPtr[r + 1] = uint32_t(cols.size());
        }
    }
    return finish(M, M, rowPtr, cols, vals, out);
}

int gen_rmat(uint64_t seed, uint32_t scale, uint32_t degree, cute_csr *out)
{
    if (scale < 4 || scale > 26 || degree == 0) return CUTE_ERR_SHAPE;
    const uint32_t n = 1u << scale;
    const uint64_t draws = uint64_t(n) * degree;
    std::vector<uint64_t> keys(draws * 2 + n);
    parallel_ranges(draws, 1 << 14, [&](uint64_t eb, uint64_t ee, unsigned) {
        for (uint64_t e = eb; e < ee; ++e) {
            uint32_t i = 0, j = 0;
            for (uint32_t lvl = 0; lvl < scale; ++lvl) {
                const float u = u01(rng_at(seed, kPattern, e * 32 + lvl));
                // quadrant probabilities a=.57 (0,0)  b=.19 (0,1)  c=.19 (1,0)  d=.05 (1,1)
                uint32_t bi, bj;
                if (u < 0.57f) { bi = 0; bj = 0; }
                else if (u < 0.76f) { bi = 0; bj = 1; }
                else if (u < 0.95f) { bi = 1; bj = 0; }
                else { bi = 1; bj = 1; }
                i = (i << 1) | bi;
                j = (j << 1) | bj;
            }
            keys[2 * e] = (uint64_t(i) << 32) | j;
            keys[2 * e + 1] = (uint64_t(j) << 32) | i;
        }
    });
    for (uint32_t i = 0; i < n; ++i) keys[draws * 2 + i] = (uint64_t(i) << 32) | i;
    std::sort(keys.begin(), keys.end());
    keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
    if (keys.size() > 0xFFFFFFFFull) return CUTE_ERR_SHAPE;
    std::vector<uint32_t> rowPtr(uint64_t(n) + 1, 0), cols(keys.size());
    std::vector<float> vals(keys.size());
    for (uint64_t k : keys) rowPtr[(k >> 32) + 1]++;
    for (uint32_t i = 0; i < n; ++i) rowPtr[i + 1] += rowPtr[i];
    for (size_t q = 0; q < keys.size(); ++q) {
        const uint32_t i = uint32_t(keys[q] >> 32), j = uint32_t(keys[q]);
        const float di = float(rowPtr[i + 1] - rowPtr[i]), dj = float(rowPtr[j + 1] - rowPtr[j]);
        cols[q] = j;
        vals[q] = 1.0f / std::sqrt(di * dj);
    }
    return finish(n, n, rowPtr, cols, vals, out);
}

}  // namespace

extern "C" int cute_gen_matrix(int kind, uint64_t seed, uint32_t p0, uint32_t p1, uint32_t p2, cute_csr *out)
{
    if (!out) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    switch (kind) {
        case 1: {
            const uint32_t M = p0;
            return gen_fixed_degree(seed, M, p1, [M](uint32_t, uint32_t &lo, uint32_t &hi) { lo = 0; hi = M - 1; }, out);
        }
        case 2: return gen_stencil(seed, p0, out);
        case 3: return gen_fem(seed, p0, p1, out);
        case 4: return gen_rmat(seed, p0, p1, out);
        case 5: {
            const uint32_t M = p0, half = p2;
            return gen_fixed_degree(seed, M, p1, [M, half](uint32_t r, uint32_t &lo, uint32_t &hi) {
                lo = r > half ? r - half : 0;
                hi = uint32_t(std::min<uint64_t>(uint64_t(M) - 1, uint64_t(r) + half));
            }, out);
        }
        default: return CUTE_ERR_ARG;
    }
}

extern "C" int cute_gen_dense(uint64_t seed, int dist, uint64_t count, float *dst)
{
    if (!dst || dist < 0 || dist > 2) return CUTE_ERR_ARG;
    parallel_ranges(count, 1 << 16, [&](uint64_t b, uint64_t e, unsigned) {
        for (uint64_t i = b; i < e; ++i) {
            const uint64_t h = rng_at(seed, kDense, i);
            if (dist == 0) dst[i] = u01(h);
            else if (dist == 1) dst[i] = sym_unit(h);
            else {
                // Box-Muller on two 24-bit uniforms taken from one 64-bit draw
                const double u1 = (double((h >> 40) & 0xFFFFFF) + 1.0) / 16777216.0;   // (0,1]
                const double u2 = double((h >> 16) & 0xFFFFFF) / 16777216.0;          // [0,1)
                dst[i] = float(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
            }
        }
    });
    return CUTE_OK;
}
