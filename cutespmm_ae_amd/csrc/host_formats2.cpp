// Host side of libcutespmm, second API family: COO loader, COO->CSR, BCSR, Blocked-ELL,
// heavy/light splitter, block classifier, double-precision CPU SpMM.  Behaviour follows
// inc/SparseCoo.hpp, inc/CSR.hpp, inc/prepareBlkEll.hpp, inc/splitter.hpp, inc/preprocess.hpp
// and inc/SPMM.cuh:123-187 of the reference; data structures are sort-based and parallel over
// block rows instead of nested hash maps.
#include <chrono>
#include <cstdio>
#include <numeric>
#include <string>

#include "common.hpp"

using namespace cute;

namespace {

struct LineCursor {
    const char *p, *end;
    bool next(const char *&b, const char *&e)
    {
        if (p >= end) return false;
        b = p;
        const char *nl = static_cast<const char *>(std::memchr(p, '\n', size_t(end - p)));
        e = nl ? nl : end;
        p = nl ? nl + 1 : end;
        return true;
    }
};

bool read_file(const char *path, std::vector<char> &buf)
{
    FILE *f = std::fopen(path, "rb");
    if (!f) return false;
    std::fseek(f, 0, SEEK_END);
    long n = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    if (n <= 0) { std::fclose(f); return false; }
    buf.resize(size_t(n) + 1);
    size_t got = std::fread(buf.data(), 1, size_t(n), f);
    std::fclose(f);
    buf[got] = '\0';
    buf.resize(got + 1);
    return got == size_t(n);
}

// Sorted distinct block columns of the rows [r0, r1) plus the nonzero count of each.
void block_row_census(const cute_csr_i32 *a, int r0, int r1, int width, std::vector<int> &ids, std::vector<int> &counts,
                      std::vector<int> &scratch)
{
    scratch.clear();
    for (int r = r0; r < r1; ++r)
        for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) scratch.push_back(a->cols[e] / width);
    std::sort(scratch.begin(), scratch.end());
    ids.clear();
    counts.clear();
    for (size_t i = 0; i < scratch.size();) {
        size_t j = i;
        while (j < scratch.size() && scratch[j] == scratch[i]) ++j;
        ids.push_back(scratch[i]);
        counts.push_back(int(j - i));
        i = j;
    }
}

bool csr_ok(const cute_csr_i32 *a) { return a && a->rowPtr && a->nrows >= 0 && a->ncols > 0 && (a->nnz == 0 || (a->cols && a->values)); }

}  // namespace

extern "C" {

void cute_coo_release(cute_coo *c)
{
    if (!c) return;
    std::free(c->rows);
    std::free(c->cols);
    std::free(c->values);
    std::memset(c, 0, sizeof(*c));
}

void cute_csr_i32_release(cute_csr_i32 *c)
{
    if (!c) return;
    std::free(c->rowPtr);
    std::free(c->cols);
    std::free(c->values);
    std::memset(c, 0, sizeof(*c));
}

int cute_coo_read(const char *path, cute_coo *out)
{
    if (!path || !out) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    std::vector<char> buf;
    if (!read_file(path, buf)) return CUTE_ERR_IO;
    LineCursor lc{buf.data(), buf.data() + buf.size() - 1};
    const char *b, *e;
    if (!lc.next(b, e)) return CUTE_ERR_IO;
    // SparseCoo.hpp:113 searches the first line for "symmetric" and mirrors with the same value.  With a
    // proper banner the line is tokenised instead: skew-symmetric files mirror with the opposite sign,
    // dense ("array") files are read, complex and hermitian files are refused (the reference would keep
    // their real parts and say nothing).
    const MmBanner bn = parse_mm_banner(b, e);
    if (bn.present && (!bn.valid || bn.field == 3 || bn.symmetry == 3)) return CUTE_ERR_FORMAT;
    const bool symmetric = bn.present ? bn.symmetry != 0 : std::string(b, e).find("symmetric") != std::string::npos;
    const float mirror_sign = (bn.present && bn.symmetry == 2) ? -1.0f : 1.0f;
    bool have = false;
    while (lc.next(b, e)) {                                                            // :119-125
        if (b < e && *b == '%') continue;
        have = true;
        break;
    }
    if (!have) return CUTE_ERR_IO;
    long long dy = 0, dx = 0, hdr = 0;
    {
        char *p = const_cast<char *>(b), *q;
        dy = std::strtoll(p, &q, 10); if (q == p) return CUTE_ERR_IO; p = q;
        dx = std::strtoll(p, &q, 10); if (q == p) return CUTE_ERR_IO; p = q;
        if (!bn.array) {
            // (the count must stand on the size line itself: strtoll would walk on into the next line)
            while (p < e && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
            if (p >= e) return CUTE_ERR_FORMAT;
            hdr = std::strtoll(p, &q, 10);
            if (q == p) return CUTE_ERR_IO;
        }
    }
    if (dy <= 0 || dx <= 0 || dy > 0x7FFFFFFF || dx > 0x7FFFFFFF || hdr < 0 || hdr > 0x7FFFFFFF) return CUTE_ERR_SHAPE;
    if (bn.present && symmetric && dy != dx) return CUTE_ERR_FORMAT;
    struct Pt { int r, c; float v; };
    std::vector<Pt> pts;
    // (an entry takes at least four bytes of the file: a forged count must not size the allocation)
    pts.reserve(std::min<size_t>(size_t(hdr), buf.size() / 4) * (symmetric ? 2 : 1));
    long long seen = 0;
    if (bn.array) {
        // column-major, one value per line; symmetric: lower triangle with, skew-symmetric without the diagonal
        long long r = bn.symmetry == 2 ? 2 : 1, c = 1;
        while (lc.next(b, e)) {
            const char *w = b;
            while (w < e && (*w == ' ' || *w == '\t' || *w == '\r')) ++w;
            if (w >= e || *w == '%') continue;
            if (c > dx || r > dy) return CUTE_ERR_FORMAT;
            char *q;
            const double d = std::strtod(w, &q);
            if (q == w) return CUTE_ERR_IO;
            if (d != 0.0) {
                pts.push_back(Pt{int(r - 1), int(c - 1), float(d)});
                if (symmetric && r != c) pts.push_back(Pt{int(c - 1), int(r - 1), mirror_sign * float(d)});
            }
            if (++r > dy) { ++c; r = bn.symmetry == 0 ? 1 : bn.symmetry == 1 ? c : c + 1; }
        }
        if (!(bn.symmetry == 2 ? c >= dx : c == dx + 1)) return CUTE_ERR_FORMAT;
    }
    while (!bn.array && lc.next(b, e)) {                                               // :130-150
        // tokens are taken from this line only (strto* would skip a newline as white space)
        auto skip = [&](char *s) { while (s < e && (*s == ' ' || *s == '\t' || *s == '\r')) ++s; return s; };
        char *p = skip(const_cast<char *>(b)), *q;
        if (p >= e) continue;            // blank line
        long long x = std::strtoll(p, &q, 10);
        if (q == p) return CUTE_ERR_IO;
        p = skip(q);
        if (p >= e) return CUTE_ERR_IO;
        long long y = std::strtoll(p, &q, 10);
        if (q == p) return CUTE_ERR_IO;
        p = skip(q);
        double v = 1.0;                                                                // :134-139
        if (p < e) {
            double d = std::strtod(p, &q);
            if (q != p) v = d;
        }
        if (x < 1 || x > dy || y < 1 || y > dx) return CUTE_ERR_RANGE;
        pts.push_back(Pt{int(x - 1), int(y - 1), float(v)});
        if (symmetric && x != y) {
            if (y > dy || x > dx) return CUTE_ERR_RANGE;
            pts.push_back(Pt{int(y - 1), int(x - 1), mirror_sign * float(v)});
        }
        ++seen;
    }
    // SparseCoo.hpp:128-149 reads every line but takes nnz from the size line, so a file whose entries do
    // not match its own size line leaves it with arrays and a count that disagree; such a file is refused here
    if (!bn.array && seen != hdr) return CUTE_ERR_FORMAT;
    if (pts.size() > 0x7FFFFFFFull) return CUTE_ERR_SHAPE;
    std::stable_sort(pts.begin(), pts.end(), [](const Pt &a, const Pt &b2) {           // :152
        return a.r != b2.r ? a.r < b2.r : a.c < b2.c;
    });
    out->dimY = int32_t(dy);
    out->dimX = int32_t(dx);
    out->nnz = int32_t(pts.size());
    out->rows = alloc_array<int32_t>(pts.size());
    out->cols = alloc_array<int32_t>(pts.size());
    out->values = alloc_array<float>(pts.size());
    if (!out->rows || !out->cols || !out->values) { cute_coo_release(out); return CUTE_ERR_NOMEM; }
    for (size_t i = 0; i < pts.size(); ++i) { out->rows[i] = pts[i].r; out->cols[i] = pts[i].c; out->values[i] = pts[i].v; }
    return CUTE_OK;
}

// Adds up entries that share a (row, column) position, in the order the array holds them (for a file
// just read: file order), after a stable sort by (row, column); nnz shrinks.  The reference keeps
// duplicates as they are (SparseCoo.hpp:130-152), and so does cute_coo_read.
int cute_coo_merge_duplicates(cute_coo *c)
{
    if (!c || c->nnz < 0 || (c->nnz && (!c->rows || !c->cols || !c->values))) return CUTE_ERR_ARG;
    const size_t n = size_t(c->nnz);
    std::vector<int> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [c](int a, int b) {
        return c->rows[a] != c->rows[b] ? c->rows[a] < c->rows[b] : c->cols[a] < c->cols[b];
    });
    std::vector<int32_t> r(n), cl(n);
    std::vector<float> v(n);
    size_t w = 0;
    for (size_t i = 0; i < n; ++i) {
        const int o = order[i];
        if (w && r[w - 1] == c->rows[o] && cl[w - 1] == c->cols[o]) v[w - 1] += c->values[o];
        else { r[w] = c->rows[o]; cl[w] = c->cols[o]; v[w] = c->values[o]; ++w; }
    }
    std::copy(r.begin(), r.begin() + w, c->rows);
    std::copy(cl.begin(), cl.begin() + w, c->cols);
    std::copy(v.begin(), v.begin() + w, c->values);
    c->nnz = int32_t(w);
    return CUTE_OK;
}

int cute_coo_save_mtx(const cute_coo *c, const char *path)
{
    if (!c || !path) return CUTE_ERR_ARG;
    FILE *f = std::fopen(path, "w");
    if (!f) return CUTE_ERR_IO;
    if (c->nnz > 0) {                                                                  // SparseCoo.hpp:275-283
        std::fprintf(f, "%%%%MatrixMarket matrix coordinate real general\n%d %d %d\n", c->dimY, c->dimX, c->nnz);
        for (int i = 0; i < c->nnz; ++i) std::fprintf(f, "%d %d %.9g\n", 1 + c->rows[i], 1 + c->cols[i], double(c->values[i]));
    }
    return std::fclose(f) == 0 ? CUTE_OK : CUTE_ERR_IO;
}

int cute_coo_to_csr(const cute_coo *c, cute_csr_i32 *out)
{
    if (!c || !out || c->dimY < 0 || c->nnz < 0) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    for (int i = 0; i < c->nnz; ++i)
        if (c->rows[i] < 0 || c->rows[i] >= c->dimY || c->cols[i] < 0 || c->cols[i] >= c->dimX) return CUTE_ERR_RANGE;
    std::vector<int> order(static_cast<size_t>(c->nnz), 0);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [c](int a, int b) {                   // CSR.hpp:166 (sortCSR)
        return c->rows[a] != c->rows[b] ? c->rows[a] < c->rows[b] : c->cols[a] < c->cols[b];
    });
    out->nrows = c->dimY;
    out->ncols = c->dimX;
    out->nnz = c->nnz;
    out->rowPtr = alloc_array<int32_t>(size_t(c->dimY) + 1);
    out->cols = alloc_array<int32_t>(size_t(c->nnz));
    out->values = alloc_array<float>(size_t(c->nnz));
    if (!out->rowPtr || !out->cols || !out->values) { cute_csr_i32_release(out); return CUTE_ERR_NOMEM; }
    for (int i = 0; i < c->nnz; ++i) {                                                 // CSR.hpp:176-186
        out->values[i] = c->values[order[i]];
        out->cols[i] = c->cols[order[i]];
        out->rowPtr[c->rows[order[i]] + 1]++;
    }
    for (int i = 0; i < c->dimY; ++i) out->rowPtr[i + 1] += out->rowPtr[i];
    return CUTE_OK;
}

int cute_csr_to_dense(const cute_csr_i32 *a, float *dense)
{
    if (!csr_ok(a) || !dense) return CUTE_ERR_ARG;
    parallel_ranges(uint64_t(a->nrows), 256, [&](uint64_t rb, uint64_t re, unsigned) {
        for (uint64_t r = rb; r < re; ++r)
            for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) dense[r * uint64_t(a->ncols) + uint64_t(a->cols[e])] = a->values[e];
    });
    return CUTE_OK;
}

int64_t cute_csr_count_blocks(const cute_csr_i32 *a, int32_t R, int32_t C)
{
    if (!csr_ok(a) || R <= 0 || C <= 0) return CUTE_ERR_ARG;
    const int nbr = (a->nrows + R - 1) / R;
    std::vector<int64_t> part(host_threads() + 1, 0);
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned t) {
        std::vector<int> ids, counts, scratch;
        int64_t n = 0;
        for (uint64_t br = bb; br < be; ++br) {
            block_row_census(a, int(br) * R, std::min(a->nrows, int(br + 1) * R), C, ids, counts, scratch);
            n += int64_t(ids.size());
        }
        part[t] = n;
    });
    return std::accumulate(part.begin(), part.end(), int64_t(0));
}

void cute_bcsr_release(cute_bcsr *b)
{
    if (!b) return;
    std::free(b->rowPtr);
    std::free(b->cols);
    std::free(b->values);
    std::memset(b, 0, sizeof(*b));
}

int cute_csr_to_bcsr(const cute_csr_i32 *a, int32_t R, int32_t C, cute_bcsr *out)
{
    if (!csr_ok(a) || !out || R <= 0 || C <= 0) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    if (a->nrows % R || a->ncols % C) return CUTE_ERR_SHAPE;                           // CSR.hpp:762-763
    const int nbr = a->nrows / R;
    // Block order inside a block row is order of first appearance while the rows are walked top
    // down, columns ascending (CSR.hpp:786-801) -- not sorted by block column.
    std::vector<std::vector<int>> order{static_cast<size_t>(nbr)};
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        std::vector<int> seen;
        for (uint64_t br = bb; br < be; ++br) {
            std::vector<int> &o = order[br];
            for (int r = int(br) * R; r < int(br + 1) * R; ++r)
                for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) {
                    const int bj = a->cols[e] / C;
                    if (std::find(o.begin(), o.end(), bj) == o.end()) o.push_back(bj);
                }
        }
    });
    out->R = R;
    out->C = C;
    out->nrows = nbr;
    out->ncols = a->ncols / C;
    out->rowPtr = alloc_array<int32_t>(size_t(nbr) + 1);
    if (!out->rowPtr) return CUTE_ERR_NOMEM;
    for (int br = 0; br < nbr; ++br) out->rowPtr[br + 1] = out->rowPtr[br] + int(order[size_t(br)].size());
    out->nblks = out->rowPtr[nbr];
    out->cols = alloc_array<int32_t>(size_t(out->nblks));
    out->values = alloc_array<float>(size_t(out->nblks) * size_t(R) * size_t(C));
    if (!out->cols || !out->values) { cute_bcsr_release(out); return CUTE_ERR_NOMEM; }
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        for (uint64_t br = bb; br < be; ++br) {
            const std::vector<int> &o = order[br];
            const int base = out->rowPtr[br];
            for (size_t i = 0; i < o.size(); ++i) out->cols[size_t(base) + i] = o[i];
            for (int r = 0; r < R; ++r) {
                const int row = int(br) * R + r;
                for (int e = a->rowPtr[row]; e < a->rowPtr[row + 1]; ++e) {
                    const int bj = a->cols[e] / C, c = a->cols[e] % C;
                    const size_t slot = size_t(std::find(o.begin(), o.end(), bj) - o.begin());
                    out->values[(size_t(base) + slot) * size_t(R) * size_t(C) + size_t(C) * size_t(r) + size_t(c)] += a->values[e];
                }
            }
        }
    });
    return CUTE_OK;
}

void cute_blocked_ell_release(cute_blocked_ell *e)
{
    if (!e) return;
    std::free(e->ellColIdx);
    std::free(e->ellValues);
    std::memset(e, 0, sizeof(*e));
}

int cute_blocked_ell_build(const cute_csr_i32 *a, int32_t B, cute_blocked_ell *out)
{
    if (!csr_ok(a) || !out || B <= 0) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    const int H = (a->nrows + B - 1) / B;                                               // prepareBlkEll.hpp:41-46,72
    std::vector<std::vector<int>> ids{static_cast<size_t>(H)};
    parallel_ranges(uint64_t(H), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        std::vector<int> counts, scratch;
        for (uint64_t br = bb; br < be; ++br)
            block_row_census(a, int(br) * B, std::min(a->nrows, int(br + 1) * B), B, ids[br], counts, scratch);
    });
    size_t W = 0, blocks = 0;
    for (const auto &v : ids) { W = std::max(W, v.size()); blocks += v.size(); }        // :75-81
    const uint64_t idx_size = uint64_t(H) * W, val_size = idx_size * uint64_t(B) * uint64_t(B);
    if (val_size > (1ull << 34)) return CUTE_ERR_NOMEM;                                  // 64 GiB of floats: refuse
    out->blockSize = B;
    out->height = H;
    out->width = int32_t(W);
    out->numBlocks = int32_t(blocks);
    out->numElems = a->nnz;
    out->ellColIdx = alloc_array<int32_t>(idx_size);
    out->ellValues = alloc_array<float>(val_size);
    if (!out->ellColIdx || !out->ellValues) { cute_blocked_ell_release(out); return CUTE_ERR_NOMEM; }
    std::fill(out->ellColIdx, out->ellColIdx + idx_size, -1);                            // :86
    parallel_ranges(uint64_t(H), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        for (uint64_t br = bb; br < be; ++br) {
            const std::vector<int> &v = ids[br];
            std::copy(v.begin(), v.end(), out->ellColIdx + br * W);
            const int r1 = std::min(a->nrows, int(br + 1) * B);
            for (int r = int(br) * B; r < r1; ++r)
                for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) {
                    const int bc = a->cols[e] / B;
                    const size_t eidx = size_t(std::lower_bound(v.begin(), v.end(), bc) - v.begin());   // find_EIdx, :159-183
                    out->ellValues[uint64_t(W) * B * uint64_t(r) + eidx * size_t(B) + size_t(a->cols[e] % B)] = a->values[e];   // :145
                }
        }
    });
    return CUTE_OK;
}

int cute_blocked_ell_to_dense(const cute_blocked_ell *e, int32_t ncols, float *dense)
{
    if (!e || !dense || !e->ellColIdx) return CUTE_ERR_ARG;
    const int B = e->blockSize, W = e->width;
    for (int br = 0; br < e->height; ++br)
        for (int bc = 0; bc < W; ++bc) {
            const int actual = e->ellColIdx[size_t(br) * size_t(W) + size_t(bc)];
            if (actual < 0) continue;
            if ((actual + 1) * B > ncols) return CUTE_ERR_RANGE;
            for (int r = br * B; r < (br + 1) * B; ++r)
                std::memcpy(dense + size_t(r) * size_t(ncols) + size_t(actual) * size_t(B),
                            e->ellValues + size_t(r) * size_t(W) * size_t(B) + size_t(bc) * size_t(B), size_t(B) * sizeof(float));
        }
    return CUTE_OK;
}

void cute_split_release(cute_split *s)
{
    if (!s) return;
    cute_coo_release(&s->heavy);
    cute_coo_release(&s->light);
    std::memset(s, 0, sizeof(*s));
}

int cute_splitter_split(const cute_csr_i32 *a, int32_t tile, int32_t thr, cute_split *out)
{
    if (!csr_ok(a) || !out || tile <= 0) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    const int nbr = (a->nrows + tile - 1) / tile;
    std::vector<uint8_t> heavy(static_cast<size_t>(a->nnz), uint8_t(0));
    struct Part { int tiles = 0, heavy_tiles = 0, light_tiles = 0; };
    std::vector<Part> part(host_threads() + 1);
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned t) {
        std::vector<int> ids, counts, scratch;
        Part p;
        for (uint64_t br = bb; br < be; ++br) {
            const int r0 = int(br) * tile, r1 = std::min(a->nrows, int(br + 1) * tile);
            block_row_census(a, r0, r1, tile, ids, counts, scratch);
            p.tiles += int(ids.size());
            for (int c : counts) (c < thr ? p.light_tiles : p.heavy_tiles)++;            // splitter.hpp:71-80
            for (int r = r0; r < r1; ++r)
                for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) {
                    const size_t k = size_t(std::lower_bound(ids.begin(), ids.end(), a->cols[e] / tile) - ids.begin());
                    heavy[size_t(e)] = counts[k] >= thr;                                  // :100-112
                }
        }
        part[t] = p;
    });
    for (const Part &p : part) { out->totalTiles += p.tiles; out->numHeavyTiles += p.heavy_tiles; out->numLightTiles += p.light_tiles; }
    for (uint8_t h : heavy) (h ? out->numHeavyElems : out->numLightElems)++;
    cute_coo *dst[2] = {&out->light, &out->heavy};
    const int cnt[2] = {out->numLightElems, out->numHeavyElems};
    for (int k = 0; k < 2; ++k) {
        dst[k]->dimY = a->nrows;
        dst[k]->dimX = a->ncols;
        dst[k]->nnz = cnt[k];
        dst[k]->rows = alloc_array<int32_t>(size_t(cnt[k]));
        dst[k]->cols = alloc_array<int32_t>(size_t(cnt[k]));
        dst[k]->values = alloc_array<float>(size_t(cnt[k]));
        if (!dst[k]->rows || !dst[k]->cols || !dst[k]->values) { cute_split_release(out); return CUTE_ERR_NOMEM; }
    }
    int fill[2] = {0, 0};
    for (int r = 0; r < a->nrows; ++r)
        for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) {                           // Insert_Next in CSR order
            const int k = heavy[size_t(e)];
            dst[k]->rows[fill[k]] = r;
            dst[k]->cols[fill[k]] = a->cols[e];
            dst[k]->values[fill[k]] = a->values[e];
            fill[k]++;
        }
    return CUTE_OK;
}

int cute_classify_blocks(const cute_csr_i32 *a, int32_t B, float dev_thr, float dominance, cute_block_class **out, int64_t *count)
{
    if (!csr_ok(a) || !out || !count || B < 4 || B % 4) return CUTE_ERR_ARG;
    *out = nullptr;
    *count = 0;
    const int nbr = (a->nrows + B - 1) / B, bands_per_block = B / 4;
    std::vector<std::vector<cute_block_class>> rows_out{static_cast<size_t>(nbr)};
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        struct Ev { int bc, kind; };   // kind 0: nonzero, 1: underloaded band, 2: overloaded band
        std::vector<Ev> ev;
        for (uint64_t br = bb; br < be; ++br) {
            ev.clear();
            const int r1 = std::min(a->nrows, int(br + 1) * B);
            for (int row = int(br) * B; row < r1; ++row) {
                int prev_band = 0, prev_nnz = 0;                                          // preprocess.hpp:78-79
                for (int e = a->rowPtr[row]; e < a->rowPtr[row + 1]; ++e) {
                    const int col = a->cols[e], band = col / 4;
                    if (band != prev_band) {
                        if (prev_nnz < 2) ev.push_back(Ev{prev_band / bands_per_block, 1});       // :87-97
                        else if (prev_nnz > 2) ev.push_back(Ev{prev_band / bands_per_block, 2});   // :98-108
                        for (int bi = prev_band + 1; bi < band; ++bi) ev.push_back(Ev{bi / bands_per_block, 1});   // :110-122
                        prev_band = band;
                        prev_nnz = 1;
                    } else {
                        prev_nnz++;
                    }
                    ev.push_back(Ev{col / B, 0});
                }
            }
            std::stable_sort(ev.begin(), ev.end(), [](const Ev &x, const Ev &y) { return x.bc < y.bc; });
            for (size_t i = 0; i < ev.size();) {
                cute_block_class b{int32_t(br), ev[i].bc, 0, 0, 0, 1};
                size_t j = i;
                for (; j < ev.size() && ev[j].bc == ev[i].bc; ++j) {
                    if (ev[j].kind == 0) b.nnz++;
                    else if (ev[j].kind == 1) b.underloads++;
                    else b.overloads++;
                }
                i = j;
                if (b.nnz == 0) continue;                                                  // only non-empty blocks are kept (:156-167)
                const float distance = 4.0f * (float(b.underloads) + float(b.overloads)) / float(B * B);
                const float ratio = (b.underloads + b.overloads) == 0 ? 0.0f : float(b.underloads) / float(b.underloads + b.overloads);
                if (distance > dev_thr && ratio <= dominance) b.kind = 0;                  // :179-186
                else if (distance > dev_thr && ratio > dominance) b.kind = 2;
                else b.kind = 1;
                rows_out[br].push_back(b);
            }
        }
    });
    size_t total = 0;
    for (const auto &v : rows_out) total += v.size();
    cute_block_class *res = alloc_array<cute_block_class>(total);
    if (!res) return CUTE_ERR_NOMEM;
    size_t k = 0;
    for (const auto &v : rows_out)
        for (const auto &b : v) res[k++] = b;
    *out = res;
    *count = int64_t(total);
    return CUTE_OK;
}

// The split the classifier implies (inc/preprocess.hpp:196-283 builds three containers from it): entries of
// blocks classified dense or 2:4-sparse form the part for the matrix cores, entries of very sparse blocks the
// remainder.  Same containers and CSR-order filling as the Splitter's.
int cute_split_by_class(const cute_csr_i32 *a, int32_t B, float dev_thr, float dominance, cute_split *out)
{
    if (!csr_ok(a) || !out || B < 4 || B % 4) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    cute_block_class *cls = nullptr;
    int64_t n = 0;
    int rc = cute_classify_blocks(a, B, dev_thr, dominance, &cls, &n);
    if (rc != CUTE_OK) return rc;
    const int nbr = (a->nrows + B - 1) / B;
    std::vector<int64_t> first(size_t(nbr) + 1, n);          // blocks are sorted by (blockRow, blockCol)
    for (int64_t i = n - 1; i >= 0; --i) first[size_t(cls[i].blockRow)] = i;
    for (int br = nbr - 1; br >= 0; --br) first[size_t(br)] = std::min(first[size_t(br)], first[size_t(br) + 1]);
    out->totalTiles = int32_t(n);
    for (int64_t i = 0; i < n; ++i) (cls[i].kind == 2 ? out->numLightTiles : out->numHeavyTiles)++;
    std::vector<uint8_t> heavy(static_cast<size_t>(a->nnz), uint8_t(0));
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        for (uint64_t br = bb; br < be; ++br) {
            const cute_block_class *lo = cls + first[br], *hi = cls + first[br + 1];
            const int r1 = std::min(a->nrows, int(br + 1) * B);
            for (int r = int(br) * B; r < r1; ++r)
                for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) {
                    const int bc = a->cols[e] / B;
                    const cute_block_class *it = std::lower_bound(lo, hi, bc, [](const cute_block_class &x, int c) { return x.blockCol < c; });
                    heavy[size_t(e)] = (it != hi && it->blockCol == bc && it->kind != 2) ? 1 : 0;
                }
        }
    });
    std::free(cls);
    for (uint8_t h : heavy) (h ? out->numHeavyElems : out->numLightElems)++;
    cute_coo *dst[2] = {&out->light, &out->heavy};
    const int cnt[2] = {out->numLightElems, out->numHeavyElems};
    for (int k = 0; k < 2; ++k) {
        dst[k]->dimY = a->nrows;
        dst[k]->dimX = a->ncols;
        dst[k]->nnz = cnt[k];
        dst[k]->rows = alloc_array<int32_t>(size_t(cnt[k]));
        dst[k]->cols = alloc_array<int32_t>(size_t(cnt[k]));
        dst[k]->values = alloc_array<float>(size_t(cnt[k]));
        if (!dst[k]->rows || !dst[k]->cols || !dst[k]->values) { cute_split_release(out); return CUTE_ERR_NOMEM; }
    }
    int fill[2] = {0, 0};
    for (int r = 0; r < a->nrows; ++r)
        for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) {
            const int k = heavy[size_t(e)];
            dst[k]->rows[fill[k]] = r;
            dst[k]->cols[fill[k]] = a->cols[e];
            dst[k]->values[fill[k]] = a->values[e];
            fill[k]++;
        }
    return CUTE_OK;
}

float cute_sequential_spmm(const cute_csr_i32 *a, const double *vals, const double *B, double *C, int32_t m, int32_t k, int32_t n)
{
    (void)k;
    if (!a || !a->rowPtr || !vals || !B || !C || m > a->nrows) return float(CUTE_ERR_ARG);
    auto t0 = std::chrono::steady_clock::now();
    for (int row = 0; row < m; ++row)
        for (int col = 0; col < n; ++col) {
            double sum = 0;
            for (int e = a->rowPtr[row]; e < a->rowPtr[row + 1]; ++e) sum += vals[e] * B[size_t(n) * size_t(a->cols[e]) + size_t(col)];
            C[size_t(n) * size_t(row) + size_t(col)] = sum;
        }
    return std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

// GET_STATS, gpu_kernels.cu:1049-1137.  The reference keys its hash maps with r_blk * (ncols / blocksize) + c_blk
// (:1064-1067); when blocksize does not divide ncols the last block column of block row i therefore shares its key
// with block (i + 1, 0), and with ncols < blocksize every block shares key 0.  Both are reproduced: the two
// blocks count as one, their rows and columns (disjoint sets) add.  Terms are added in key order, in float.
int cute_block_stats(const cute_csr_i32 *a, int32_t blocksize, float *stats)
{
    if (!csr_ok(a) || !stats || blocksize <= 0) return CUTE_ERR_ARG;
    const int bs = blocksize, nbr = (a->nrows + bs - 1) / bs;
    const uint64_t per_row = uint64_t(a->ncols) / uint64_t(bs);
    if ((uint64_t(nbr) + 1) * per_row + per_row >= (uint64_t(1) << 32)) return CUTE_ERR_SHAPE;   // 32-bit keys would wrap
    struct Blk { int bc, nnz, rows, cols; };
    std::vector<std::vector<Blk>> per{static_cast<size_t>(nbr)};
    parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned) {
        std::vector<std::pair<int, int>> ent;          // (column, row inside the block row)
        std::vector<int> stamp(size_t(bs), -1);
        for (uint64_t br = bb; br < be; ++br) {
            ent.clear();
            const int r0 = int(br) * bs, r1 = std::min(a->nrows, r0 + bs);
            for (int r = r0; r < r1; ++r)
                for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) ent.emplace_back(a->cols[e], r - r0);
            std::sort(ent.begin(), ent.end());
            std::fill(stamp.begin(), stamp.end(), -1);
            std::vector<Blk> &out = per[br];
            for (size_t i = 0; i < ent.size();) {
                const int bc = per_row ? ent[i].first / bs : 0;
                Blk b{bc, 0, 0, 0};
                size_t j = i;
                for (; j < ent.size() && (per_row ? ent[j].first / bs : 0) == bc; ++j) {
                    b.nnz++;
                    if (j == i || ent[j].first != ent[j - 1].first) b.cols++;
                    if (stamp[size_t(ent[j].second)] != int(out.size())) { stamp[size_t(ent[j].second)] = int(out.size()); b.rows++; }
                }
                out.push_back(b);
                i = j;
            }
        }
    });
    float anrs = 0.0f, ancs = 0.0f, dens = 0.0f;
    uint32_t blocks = 0;
    auto emit = [&](const Blk &b) {
        dens += float(b.nnz) / float(bs * bs);
        anrs += float(b.nnz) / float(b.rows);
        ancs += float(b.nnz) / float(b.cols);
        ++blocks;
    };
    if (per_row == 0) {                       // every nonzero has key 0: one block, its columns need a union
        Blk all{0, 0, 0, 0};
        std::vector<char> seen(size_t(a->ncols), 0);
        for (int br = 0; br < nbr; ++br)
            for (const Blk &b : per[size_t(br)]) { all.nnz += b.nnz; all.rows += b.rows; }
        for (int e = 0; e < a->rowPtr[a->nrows]; ++e)
            if (!seen[size_t(a->cols[e])]) { seen[size_t(a->cols[e])] = 1; all.cols++; }
        if (all.nnz) emit(all);
    } else {
        Blk carry{0, 0, 0, 0};                // block (br - 1, per_row): its key is that of block (br, 0)
        for (int br = 0; br <= nbr; ++br) {
            const std::vector<Blk> empty_row;
            const std::vector<Blk> &row = br < nbr ? per[size_t(br)] : empty_row;
            size_t first = 0;
            if (carry.nnz) {
                if (!row.empty() && row[0].bc == 0) {
                    carry.nnz += row[0].nnz; carry.rows += row[0].rows; carry.cols += row[0].cols;
                    first = 1;
                }
                emit(carry);
                carry = Blk{0, 0, 0, 0};
            }
            for (size_t i = first; i < row.size(); ++i) {
                if (uint64_t(row[i].bc) == per_row) carry = row[i];
                else emit(row[i]);
            }
        }
    }
    stats[0] = anrs / float(blocks);
    stats[1] = ancs / float(blocks);
    stats[2] = float(blocks);
    stats[3] = dens / float(blocks);
    return CUTE_OK;
}

// GET_ANXS, gpu_kernels.cu:1139-1186: nonzeros per distinct (band, segment) pair.  axis != 0: bands are block
// rows, segments columns (how often a fetched B row is reused inside a row panel); axis == 0: bands are block
// columns, segments rows.
int cute_anxs(const cute_csr_i32 *a, int32_t blocksize, int32_t axis, float *out)
{
    if (!csr_ok(a) || !out || blocksize <= 0) return CUTE_ERR_ARG;
    const int bs = blocksize;
    std::vector<int64_t> part(host_threads() + 1, 0);
    if (axis) {
        const int nbr = (a->nrows + bs - 1) / bs;
        parallel_ranges(uint64_t(nbr), 8, [&](uint64_t bb, uint64_t be, unsigned t) {
            std::vector<int> c;
            int64_t n = 0;
            for (uint64_t br = bb; br < be; ++br) {
                const int r0 = int(br) * bs, r1 = std::min(a->nrows, r0 + bs);
                c.assign(a->cols + a->rowPtr[r0], a->cols + a->rowPtr[r1]);
                std::sort(c.begin(), c.end());
                n += int64_t(std::unique(c.begin(), c.end()) - c.begin());
            }
            part[t] = n;
        });
    } else {
        parallel_ranges(uint64_t(a->nrows), 256, [&](uint64_t rb, uint64_t re, unsigned t) {
            std::vector<int> c;
            int64_t n = 0;
            for (uint64_t r = rb; r < re; ++r) {
                c.clear();
                for (int e = a->rowPtr[r]; e < a->rowPtr[r + 1]; ++e) c.push_back(a->cols[e] / bs);
                std::sort(c.begin(), c.end());
                n += int64_t(std::unique(c.begin(), c.end()) - c.begin());
            }
            part[t] = n;
        });
    }
    const int64_t sum = std::accumulate(part.begin(), part.end(), int64_t(0));
    *out = float(uint32_t(a->rowPtr[a->nrows])) / float(int(sum));      // (float)nnz / sum, :1185
    return CUTE_OK;
}

}  // extern "C"
