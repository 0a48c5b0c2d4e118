// Host side of libcutespmm: MatrixMarket reader, CSR -> HRPB builder, the MFMA re-tile
// and its inverse, the launch partition and the result metrics.  Nothing here touches
// the GPU.
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <string>

#include "common.hpp"

using namespace cute;

extern "C" {

const char *cute_status_string(int s)
{
    switch (s) {
        case CUTE_OK: return "ok";
        case CUTE_ERR_IO: return "file missing, unreadable or malformed";
        case CUTE_ERR_SHAPE: return "bad shape (M, K must be multiples of 16; N > 0)";
        case CUTE_ERR_UNSORTED: return "CSR row has unsorted or duplicate columns";
        case CUTE_ERR_RANGE: return "index out of range";
        case CUTE_ERR_ARG: return "bad argument";
        case CUTE_ERR_NOMEM: return "out of memory";
        case CUTE_ERR_HIP: return "HIP runtime error";
        case CUTE_ERR_NO_DEVICE: return "no gfx950 device";
        case CUTE_ERR_FORMAT: return "format stream failed validation";
        case CUTE_ERR_SCRATCH: return "the plan's partial tiles do not fit the static scratch buffer";
        default: return "unknown status";
    }
}

void cute_free(void *p) { std::free(p); }

void cute_csr_release(cute_csr *c)
{
    if (!c) return;
    std::free(c->rowPtr);
    std::free(c->cols);
    std::free(c->vals);
    std::memset(c, 0, sizeof(*c));
}

}  // extern "C"

// ---------------------------------------------------------------------------------
// MatrixMarket reader (behaviour of IO.cu:10-87; one read of the file, parsed in memory)
// ---------------------------------------------------------------------------------
namespace {

struct LineCursor {
    const char *p, *end;
    // Next line as [b, e); false at end of buffer.
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

inline const char *skip_ws(const char *s, const char *e)
{
    while (s < e && (*s == ' ' || *s == '\t' || *s == '\r')) ++s;
    return s;
}
inline const char *skip_word(const char *s, const char *e)
{
    while (s < e && *s != ' ' && *s != '\t' && *s != '\r') ++s;
    return s;
}
// Leading integer of the next word, like std::stoi on a `>>`-extracted word.
// 1: parsed, 0: no word on the line, -1: word does not start with an integer.
inline int next_int(const char *&s, const char *e, long long &v)
{
    s = skip_ws(s, e);
    if (s >= e) return 0;
    const char *w = s;
    bool neg = false;
    if (*w == '+' || *w == '-') { neg = (*w == '-'); ++w; }
    if (w >= e || *w < '0' || *w > '9') return -1;
    long long x = 0;
    while (w < e && *w >= '0' && *w <= '9') { x = x * 10 + (*w - '0'); ++w; }
    v = neg ? -x : x;
    s = skip_word(w, e);
    return 1;
}

}  // namespace

namespace {

struct Triplet { uint32_t r, c; float v; };

// The value-keeping reader: tokenises the banner, so that skew-symmetric files mirror with the
// opposite sign, dense ("array") files are read, and fields this library has no arithmetic for
// (complex, hermitian) are refused instead of silently losing their imaginary parts.  Entries
// come out in file order, a mirrored entry right behind its original, exactly where the
// reference's loader puts them (IO.cu:71-84).  A file without a banner is read the way the
// reference reads every file: "symmetric" anywhere on the first line means mirror.
// Largest dimension a size line may state: the reference parses it with stoi (IO.cu:23-29), which throws
// beyond INT_MAX -- and a forged line must not turn into a multi-gigabyte row-pointer allocation.
constexpr long long kMaxFileDim = 0x7FFFFFFFll - 16;

int read_triplets(const char *begin, const char *end_, long long &m, long long &k, std::vector<Triplet> &out)
{
    LineCursor lc{begin, end_};
    const char *b, *e;
    if (!lc.next(b, e)) return CUTE_ERR_IO;
    const MmBanner bn = parse_mm_banner(b, e);
    bool mirror;
    float mirror_sign = 1.0f;
    if (bn.present) {
        if (!bn.valid || bn.field == 3 || bn.symmetry == 3) return CUTE_ERR_FORMAT;
        mirror = bn.symmetry != 0;
        if (bn.symmetry == 2) mirror_sign = -1.0f;
    } else {
        mirror = std::string(b, e).find("symmetric") != std::string::npos;
    }
    bool have_size = false;
    while (lc.next(b, e)) {
        if (b < e && *b == '%') continue;
        if (skip_ws(b, e) >= e) continue;
        have_size = true;
        break;
    }
    if (!have_size) return CUTE_ERR_IO;
    const char *s = b;
    if (next_int(s, e, m) != 1 || next_int(s, e, k) != 1 || m <= 0 || k <= 0) return CUTE_ERR_IO;
    if (m > kMaxFileDim || k > kMaxFileDim) return CUTE_ERR_SHAPE;
    if (mirror && bn.present && m != k) return CUTE_ERR_FORMAT;
    // a coordinate file announces its number of entries; what follows must be exactly that many
    long long announced = -1, seen = 0;
    if (!bn.array && (next_int(s, e, announced) != 1 || announced < 0)) return CUTE_ERR_FORMAT;
    auto push = [&](long long r, long long c, float v) {
        out.push_back(Triplet{uint32_t(r - 1), uint32_t(c - 1), v});
        if (mirror && r != c) out.push_back(Triplet{uint32_t(c - 1), uint32_t(r - 1), mirror_sign * v});
    };
    if (bn.array) {
        // dense, column-major, one value per line; symmetric files hold the lower triangle with,
        // skew-symmetric ones without the diagonal.  Zeros are not entries.
        long long r = bn.symmetry == 2 ? 2 : 1, c = 1;
        while (lc.next(b, e)) {
            const char *w = skip_ws(b, e);
            if (w >= e || *w == '%') continue;
            if (c > k || r > m) return CUTE_ERR_FORMAT;            // more values than the header promises
            char *endp = nullptr;
            const double d = std::strtod(w, &endp);
            if (endp == w) return CUTE_ERR_IO;
            if (d != 0.0) push(r, c, float(d));
            if (++r > m) { ++c; r = bn.symmetry == 0 ? 1 : bn.symmetry == 1 ? c : c + 1; }
        }
        const bool complete = bn.symmetry == 2 ? (c >= k) : (c == k + 1);
        return complete ? CUTE_OK : CUTE_ERR_FORMAT;
    }
    while (lc.next(b, e)) {
        long long r, c;
        s = b;
        const int g = next_int(s, e, r);
        if (g == 0) continue;                                      // blank line
        if (g < 0 || next_int(s, e, c) != 1) return CUTE_ERR_IO;
        if (r < 1 || r > m || c < 1 || c > k) return CUTE_ERR_RANGE;
        if (mirror && r != c && (c > m || r > k)) return CUTE_ERR_RANGE;
        float v = 1.0f;
        const char *w = skip_ws(s, e);
        if (w < e) {
            char *endp = nullptr;
            const double d = std::strtod(w, &endp);                // the buffer is NUL-terminated
            if (endp != w) v = static_cast<float>(d);
        }
        push(r, c, v);
        ++seen;
    }
    return seen == announced ? CUTE_OK : CUTE_ERR_FORMAT;
}

int csr_from_triplets(long long m, long long k, const std::vector<Triplet> &t, cute_csr *out)
{
    if (t.size() > 0xFFFFFFFFull) return CUTE_ERR_SHAPE;
    const uint32_t M = uint32_t((m - 1) / CUTE_TM + 1) * CUTE_TM;   // IO.cu:30
    const uint32_t K = uint32_t((k - 1) / CUTE_TK + 1) * CUTE_TK;   // IO.cu:31
    uint32_t *rowPtr = alloc_array<uint32_t>(uint64_t(M) + 1);
    uint32_t *cols = alloc_array<uint32_t>(t.size());
    float *vals = alloc_array<float>(t.size());
    if (!rowPtr || !cols || !vals) { std::free(rowPtr); std::free(cols); std::free(vals); return CUTE_ERR_NOMEM; }
    for (const Triplet &x : t) rowPtr[x.r + 1]++;
    for (uint32_t i = 0; i < M; ++i) rowPtr[i + 1] += rowPtr[i];
    std::vector<uint32_t> fill(M, 0u);
    for (const Triplet &x : t) {
        const uint32_t pos = rowPtr[x.r] + fill[x.r]++;
        cols[pos] = x.c;
        vals[pos] = x.v;
    }
    out->M = M; out->K = K; out->nnz = uint32_t(t.size());
    out->rowPtr = rowPtr; out->cols = cols; out->vals = vals;
    return CUTE_OK;
}

}  // namespace

extern "C" int cute_mtx_read(const char *path, int keep_values, cute_csr *out)
{
    if (!path || !out) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    FILE *f = std::fopen(path, "rb");
    if (!f) return CUTE_ERR_IO;
    std::fseek(f, 0, SEEK_END);
    long fsz = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    if (fsz <= 0) { std::fclose(f); return CUTE_ERR_IO; }
    std::vector<char> buf(static_cast<size_t>(fsz) + 1);
    size_t got = std::fread(buf.data(), 1, size_t(fsz), f);
    std::fclose(f);
    if (got != size_t(fsz)) return CUTE_ERR_IO;
    buf[got] = '\0';

    if (keep_values) {
        long long m = 0, k = 0;
        std::vector<Triplet> t;
        const int rc = read_triplets(buf.data(), buf.data() + got, m, k, t);
        return rc == CUTE_OK ? csr_from_triplets(m, k, t, out) : rc;
    }

    // keep_values == 0: the reference's reader, quirk for quirk.
    LineCursor lc{buf.data(), buf.data() + got};
    const char *b, *e;
    if (!lc.next(b, e)) return CUTE_ERR_IO;
    // IO.cu:16 -- only the first line is searched for "symmetric".
    bool symmetric = std::string(b, e).find("symmetric") != std::string::npos;
    bool have_size = false;
    while (lc.next(b, e)) {              // IO.cu:17-22
        if (b < e && *b == '%') continue;
        have_size = true;
        break;
    }
    if (!have_size) return CUTE_ERR_IO;
    long long m = 0, k = 0;
    const char *s = b;
    if (next_int(s, e, m) != 1 || next_int(s, e, k) != 1 || m <= 0 || k <= 0) return CUTE_ERR_IO;
    if (m > kMaxFileDim || k > kMaxFileDim) return CUTE_ERR_SHAPE;   // where the reference's stoi throws
    const uint32_t M = uint32_t((m - 1) / CUTE_TM + 1) * CUTE_TM;   // IO.cu:30
    const uint32_t K = uint32_t((k - 1) / CUTE_TK + 1) * CUTE_TK;   // IO.cu:31
    const char *data_begin = lc.p;

    uint32_t *rowPtr = alloc_array<uint32_t>(uint64_t(M) + 1);
    if (!rowPtr) return CUTE_ERR_NOMEM;
    uint64_t total = 0;
    int status = CUTE_OK;
    while (lc.next(b, e)) {              // pass 1, IO.cu:34-45
        long long r, c;
        s = b;
        int g = next_int(s, e, r);
        if (g == 0) continue;            // blank line
        if (g < 0 || next_int(s, e, c) != 1) { status = CUTE_ERR_IO; break; }
        if (r < 1 || r > m || c < 1 || c > k) { status = CUTE_ERR_RANGE; break; }
        rowPtr[r]++;
        total++;
        if (symmetric && r != c) {
            if (c > m || r > k) { status = CUTE_ERR_RANGE; break; }
            rowPtr[c]++;
            total++;
        }
    }
    if (status == CUTE_OK && total > 0xFFFFFFFFull) status = CUTE_ERR_SHAPE;
    if (status != CUTE_OK) { std::free(rowPtr); return status; }
    for (uint32_t i = 0; i < M; ++i) rowPtr[i + 1] += rowPtr[i];
    uint32_t *cols = alloc_array<uint32_t>(total);
    float *vals = alloc_array<float>(total);
    std::vector<uint32_t> fill(M, 0u);
    if (!cols || !vals) { std::free(rowPtr); std::free(cols); std::free(vals); return CUTE_ERR_NOMEM; }
    lc = LineCursor{data_begin, buf.data() + got};
    while (lc.next(b, e)) {              // pass 2, IO.cu:61-85
        long long r, c;
        s = b;
        if (next_int(s, e, r) == 0) continue;
        next_int(s, e, c);
        const uint32_t rr = uint32_t(r - 1), cc = uint32_t(c - 1);
        uint32_t pos = rowPtr[rr] + fill[rr]++;
        cols[pos] = cc;
        vals[pos] = 1.0f;                // IO.cu:68
        if (symmetric && rr != cc) {
            pos = rowPtr[cc] + fill[cc]++;
            cols[pos] = rr;
            vals[pos] = 1.0f;            // IO.cu:81
        }
    }
    out->M = M;
    out->K = K;
    out->nnz = uint32_t(total);
    out->rowPtr = rowPtr;
    out->cols = cols;
    out->vals = vals;
    return CUTE_OK;
}

// Sorts every row by column and adds up entries that share a (row, column) position, in the order
// the file held them; the arrays shrink in place and nnz follows.  For files that list an entry
// more than once (assembly output): the format builder refuses duplicate columns.
extern "C" int cute_csr_merge_duplicates(cute_csr *c)
{
    if (!c || !c->rowPtr) return CUTE_ERR_ARG;
    std::vector<std::pair<uint32_t, float>> tmp;
    uint32_t w = 0, row_start = 0;
    for (uint32_t r = 0; r < c->M; ++r) {
        const uint32_t s = row_start, e = c->rowPtr[r + 1];
        row_start = e;
        tmp.clear();
        for (uint32_t i = s; i < e; ++i) tmp.emplace_back(c->cols[i], c->vals[i]);
        std::stable_sort(tmp.begin(), tmp.end(),
                         [](const std::pair<uint32_t, float> &a, const std::pair<uint32_t, float> &b) { return a.first < b.first; });
        c->rowPtr[r] = w;
        for (size_t i = 0; i < tmp.size(); ++i) {
            if (i && tmp[i].first == tmp[i - 1].first) c->vals[w - 1] += tmp[i].second;
            else { c->cols[w] = tmp[i].first; c->vals[w] = tmp[i].second; ++w; }
        }
    }
    c->rowPtr[c->M] = w;
    c->nnz = w;
    return CUTE_OK;
}

extern "C" int cute_csr_sort_rows(cute_csr *c)
{
    if (!c || !c->rowPtr) return CUTE_ERR_ARG;
    int bad = 0;
    parallel_ranges(c->M, 256, [&](uint64_t rb, uint64_t re, unsigned) {
        std::vector<std::pair<uint32_t, float>> tmp;
        for (uint64_t r = rb; r < re; ++r) {
            uint32_t s = c->rowPtr[r], e = c->rowPtr[r + 1];
            bool sorted = true;
            for (uint32_t i = s + 1; i < e; ++i)
                if (c->cols[i] <= c->cols[i - 1]) { sorted = false; break; }
            if (sorted) continue;
            tmp.clear();
            for (uint32_t i = s; i < e; ++i) tmp.emplace_back(c->cols[i], c->vals[i]);
            std::stable_sort(tmp.begin(), tmp.end(),
                             [](const std::pair<uint32_t, float> &a, const std::pair<uint32_t, float> &b) {
                                 return a.first < b.first;
                             });
            for (uint32_t i = s; i < e; ++i) {
                c->cols[i] = tmp[i - s].first;
                c->vals[i] = tmp[i - s].second;
                if (i > s && c->cols[i] == c->cols[i - 1]) __atomic_store_n(&bad, 1, __ATOMIC_RELAXED);
            }
        }
    });
    return bad ? CUTE_ERR_UNSORTED : CUTE_OK;
}

// ---------------------------------------------------------------------------------
// CSR -> canonical HRPB (outputs of data.cu:94-335)
//
// Two parallel sweeps over the row panels instead of the reference's per-thread work
// spaces: sweep 1 finds each panel's sorted active columns and the nonzero count of each
// of its blocks; a serial prefix pass fixes every block's offset; sweep 2 writes each
// record in place.  Every word written depends only on the input, never on the thread
// count.
// ---------------------------------------------------------------------------------
namespace {

struct PanelScratch {
    std::vector<uint32_t> act;        // sorted distinct columns of the panel
    std::vector<uint16_t> blk_nnz;    // nonzeros per block (<= 256)
};

inline uint32_t record_words(uint32_t nnz_blk)
{
    uint32_t w = ((nnz_blk + 1u) / 2u) * 2u + CUTE_META_WORDS;              // data.cu:225
    return ((w + CUTE_CHUNK_WORDS - 1u) / CUTE_CHUNK_WORDS) * CUTE_CHUNK_WORDS;  // data.cu:226-227
}

}  // namespace

extern "C" void cute_hrpb_host_release(cute_hrpb_host *h)
{
    if (!h) return;
    std::free(h->blockedRowPtr);
    std::free(h->activeCols);
    std::free(h->sizePtr);
    std::free(h->blocksData);
    std::memset(h, 0, sizeof(*h));
}

extern "C" int cute_hrpb_build(uint32_t M, uint32_t K, const uint32_t *rowPtr, const uint32_t *cols,
                               const float *vals, cute_hrpb_host *out)
{
    if (!rowPtr || !out || (rowPtr[M] && (!cols || !vals))) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    if (M == 0 || K == 0 || M % CUTE_TM || K % CUTE_TK) return CUTE_ERR_SHAPE;
    const uint32_t P = M / CUTE_TM;
    std::vector<PanelScratch> panels(P);
    int status = CUTE_OK;

    // sweep 1: active columns, validation, per-block nonzero counts
    parallel_ranges(P, 16, [&](uint64_t pb, uint64_t pe, unsigned) {
        std::vector<uint32_t> tmp;
        for (uint64_t p = pb; p < pe; ++p) {
            const uint32_t r0 = uint32_t(p) * CUTE_TM;
            tmp.clear();
            for (uint32_t r = r0; r < r0 + CUTE_TM; ++r) {
                uint32_t s = rowPtr[r], e = rowPtr[r + 1];
                if (e < s) { __atomic_store_n(&status, int(CUTE_ERR_RANGE), __ATOMIC_RELAXED); return; }
                for (uint32_t i = s; i < e; ++i) {
                    if (cols[i] >= K) { __atomic_store_n(&status, int(CUTE_ERR_RANGE), __ATOMIC_RELAXED); return; }
                    if (i > s && cols[i] <= cols[i - 1]) {
                        __atomic_store_n(&status, int(CUTE_ERR_UNSORTED), __ATOMIC_RELAXED);
                        return;
                    }
                    tmp.push_back(cols[i]);
                }
            }
            std::sort(tmp.begin(), tmp.end());
            PanelScratch &ps = panels[p];
            ps.act = tmp;
            ps.act.erase(std::unique(ps.act.begin(), ps.act.end()), ps.act.end());
            ps.act.shrink_to_fit();
            const uint32_t nblk = uint32_t((ps.act.size() + CUTE_TK - 1) / CUTE_TK);
            ps.blk_nnz.assign(nblk, 0);
            // tmp still holds every nonzero's column (sorted, with repeats): count per block
            uint32_t ai = 0;
            for (uint32_t c : tmp) {
                while (ps.act[ai] != c) ++ai;
                ps.blk_nnz[ai / CUTE_TK]++;
            }
        }
    });
    if (status != CUTE_OK) return status;

    uint32_t *brp = alloc_array<uint32_t>(uint64_t(P) + 1);
    if (!brp) return CUTE_ERR_NOMEM;
    uint64_t nb64 = 0;
    for (uint32_t p = 0; p < P; ++p) {
        nb64 += panels[p].blk_nnz.size();
        if (nb64 > 0xFFFFFFFFull / CUTE_TK) { std::free(brp); return CUTE_ERR_SHAPE; }
        brp[p + 1] = uint32_t(nb64);
    }
    const uint32_t nb = uint32_t(nb64);
    uint64_t *sizePtr = alloc_array<uint64_t>(uint64_t(nb) + 1);
    uint32_t *acols = alloc_array<uint32_t>(uint64_t(nb) * CUTE_TK);
    if (!sizePtr || !acols) { std::free(brp); std::free(sizePtr); std::free(acols); return CUTE_ERR_NOMEM; }
    for (uint32_t p = 0; p < P; ++p)
        for (uint32_t b = 0; b < panels[p].blk_nnz.size(); ++b)
            sizePtr[brp[p] + b + 1] = sizePtr[brp[p] + b] + record_words(panels[p].blk_nnz[b]);
    const uint64_t words = sizePtr[nb];
    uint32_t *stream = alloc_array<uint32_t>(words);
    if (!stream) { std::free(brp); std::free(sizePtr); std::free(acols); return CUTE_ERR_NOMEM; }

    std::vector<uint64_t> bricks_per_thread(host_threads() + 1, 0);
    // sweep 2: write the records
    parallel_ranges(P, 16, [&](uint64_t pb, uint64_t pe, unsigned tid) {
        struct Entry { uint32_t slot; uint16_t bit; float v; };   // slot = block*4 + brick column
        std::vector<Entry> ent;
        std::vector<uint32_t> bucket_start;
        uint64_t bricks = 0;
        for (uint64_t p = pb; p < pe; ++p) {
            const PanelScratch &ps = panels[p];
            const uint32_t len = uint32_t(ps.act.size());
            if (!len) continue;
            const uint32_t nblk = uint32_t(ps.blk_nnz.size());
            const uint32_t b0 = brp[p];
            std::memcpy(acols + uint64_t(b0) * CUTE_TK, ps.act.data(), len * sizeof(uint32_t));
            // every nonzero -> (block, brick column, bit); rows ascending, columns ascending
            ent.clear();
            bucket_start.assign(uint64_t(nblk) * 4 + 1, 0);
            const uint32_t r0 = uint32_t(p) * CUTE_TM;
            for (uint32_t r = 0; r < CUTE_TM; ++r) {
                const uint32_t *lo = ps.act.data();
                for (uint32_t i = rowPtr[r0 + r]; i < rowPtr[r0 + r + 1]; ++i) {
                    lo = std::lower_bound(lo, ps.act.data() + len, cols[i]);
                    uint32_t ci = uint32_t(lo - ps.act.data());
                    uint32_t slot = (ci / CUTE_TK) * 4 + (ci % CUTE_TK) / CUTE_BRICK_K;
                    ent.push_back(Entry{slot, uint16_t(r * CUTE_BRICK_K + ci % CUTE_BRICK_K), vals[i]});
                    bucket_start[slot + 1]++;
                }
            }
            for (size_t i = 0; i + 1 < bucket_start.size(); ++i) bucket_start[i + 1] += bucket_start[i];
            for (uint32_t b = 0; b < nblk; ++b) {
                uint32_t *rec = stream + sizePtr[b0 + b];
                const uint64_t next = sizePtr[b0 + b + 1];
                std::memcpy(rec + 0, &next, 8);                                  // words 0-1
                rec[26] = uint32_t((next - sizePtr[b0 + b]) / CUTE_CHUNK_WORDS); // this record's chunks
                if (b + 1 < nblk) {
                    rec[27] = uint32_t((sizePtr[b0 + b + 2] - next) / CUTE_CHUNK_WORDS);
                    uint32_t ncol = std::min<uint32_t>(CUTE_TK, len - (b + 1) * CUTE_TK);
                    std::memcpy(rec + 8, ps.act.data() + (b + 1) * CUTE_TK, ncol * sizeof(uint32_t));
                }
                uint16_t prefix[4];
                const uint32_t base = bucket_start[b * 4];
                for (uint32_t j = 0; j < 4; ++j) prefix[j] = uint16_t(bucket_start[b * 4 + j] - base);
                std::memcpy(rec + 24, prefix, 8);                                // words 24-25
            }
            // scatter values / bits; entries of one bucket arrive in (row, k) order already
            std::vector<uint32_t> &fill = bucket_start;  // reuse as running cursor
            // (walk entries in generation order; cursor per slot)
            std::vector<uint32_t> cursor(fill.begin(), fill.end() - 1);
            for (const Entry &en : ent) {
                const uint32_t b = en.slot / 4, j = en.slot % 4;
                uint32_t *rec = stream + sizePtr[b0 + b];
                const uint32_t base = fill[b * 4];
                float *v = reinterpret_cast<float *>(rec + CUTE_META_WORDS);
                v[cursor[en.slot]++ - base] = en.v;
                uint64_t bm;
                std::memcpy(&bm, rec + 28 + 2 * j, 8);
                if (!bm) {
                    bricks++;
                    uint64_t cp;
                    std::memcpy(&cp, rec + 2, 8);
                    cp |= 1ull << (j * 4);                                        // words 2-3
                    std::memcpy(rec + 2, &cp, 8);
                }
                bm |= 1ull << en.bit;
                std::memcpy(rec + 28 + 2 * j, &bm, 8);                           // words 28-35
                rec[4 + j] += (en.bit < 32) ? 1u : (1u << 8);                    // words 4-7
            }
        }
        bricks_per_thread[tid] = bricks;
    });

    uint64_t bricks = 0;
    for (uint64_t x : bricks_per_thread) bricks += x;
    out->M = M;
    out->K = K;
    out->numRowPanels = P;
    out->numBlocks = nb;
    out->numWords = words;
    out->blockedRowPtr = brp;
    out->activeCols = acols;
    out->sizePtr = sizePtr;
    out->blocksData = stream;
    out->rowPtr = rowPtr;
    out->cols = cols;
    out->vals = vals;
    out->nnz = rowPtr[M];
    out->numBricks = uint32_t(bricks);
    return CUTE_OK;
}

// ---------------------------------------------------------------------------------
// canonical <-> MFMA-tiled
// ---------------------------------------------------------------------------------
extern "C" void cute_hrpb_tiled_release(cute_hrpb_tiled *t)
{
    if (!t) return;
    std::free(t->blockedRowPtr);
    std::free(t->hdr);
    std::free(t->vals);
    std::memset(t, 0, sizeof(*t));
}

extern "C" int cute_hrpb_retile(const cute_hrpb_host *h, cute_hrpb_tiled *out)
{
    if (!h || !out || !h->blockedRowPtr) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    const uint32_t nb = h->numBlocks;
    // value offsets: exclusive prefix of per-block nonzeros (last prefix entry + last brick popcount)
    std::vector<uint64_t> voff(uint64_t(nb) + 1, 0);
    for (uint32_t b = 0; b < nb; ++b) {
        const uint32_t *rec = h->blocksData + h->sizePtr[b];
        uint32_t n = 0;
        for (uint32_t j = 0; j < 4; ++j) {
            uint64_t bm;
            std::memcpy(&bm, rec + 28 + 2 * j, 8);
            n += uint32_t(__builtin_popcountll(bm));
        }
        voff[b + 1] = voff[b] + n;
    }
    if (voff[nb] > 0xFFFFFFFFull) return CUTE_ERR_SHAPE;
    uint32_t *hdr = alloc_array<uint32_t>(uint64_t(nb) * CUTE_TILED_HDR_WORDS);
    float *vals = alloc_array<float>(voff[nb]);
    uint32_t *brp = alloc_array<uint32_t>(uint64_t(h->numRowPanels) + 1);
    if (!hdr || !vals || !brp) { std::free(hdr); std::free(vals); std::free(brp); return CUTE_ERR_NOMEM; }
    std::memcpy(brp, h->blockedRowPtr, (uint64_t(h->numRowPanels) + 1) * sizeof(uint32_t));
    int status = CUTE_OK;
    parallel_ranges(nb, 1024, [&](uint64_t bb, uint64_t be, unsigned) {
        for (uint64_t b = bb; b < be; ++b) {
            const uint32_t *rec = h->blocksData + h->sizePtr[b];
            const float *src = reinterpret_cast<const float *>(rec + CUTE_META_WORDS);
            const uint32_t *ac = h->activeCols + b * CUTE_TK;
            uint32_t *hd = hdr + b * CUTE_TILED_HDR_WORDS;
            uint16_t prefix[4];
            std::memcpy(prefix, rec + 24, 8);
            uint32_t off = uint32_t(voff[b]);
            for (uint32_t j = 0; j < 4; ++j) {
                for (uint32_t k = 0; k < 4; ++k) hd[k * 4 + j] = ac[j * 4 + k];
                uint64_t canon;
                std::memcpy(&canon, rec + 28 + 2 * j, 8);
                const uint64_t lane = bitmap_to_lane_order(canon);
                std::memcpy(hd + 16 + 2 * j, &lane, 8);
                hd[24 + j] = off;
                if (off - uint32_t(voff[b]) != prefix[j]) __atomic_store_n(&status, int(CUTE_ERR_FORMAT), __ATOMIC_RELAXED);
                // value of canonical bit c sits at rank(c) in src; lane order wants it at rank(lane bit)
                uint64_t rest = lane;
                while (rest) {
                    unsigned lb = unsigned(__builtin_ctzll(rest));
                    rest &= rest - 1;
                    unsigned cb = (lb & 15u) * 4u + (lb >> 4);
                    unsigned crank = unsigned(__builtin_popcountll(canon & ((1ull << cb) - 1ull)));
                    vals[off++] = src[prefix[j] + crank];
                }
            }
            hd[28] = off - uint32_t(voff[b]);
        }
    });
    if (status != CUTE_OK) { std::free(hdr); std::free(vals); std::free(brp); return status; }
    out->M = h->M;
    out->K = h->K;
    out->numRowPanels = h->numRowPanels;
    out->numBlocks = nb;
    out->numVals = voff[nb];
    out->blockedRowPtr = brp;
    out->hdr = hdr;
    out->vals = vals;
    return CUTE_OK;
}

extern "C" int cute_hrpb_untile(const cute_hrpb_tiled *t, cute_hrpb_host *out)
{
    if (!t || !out || !t->blockedRowPtr) return CUTE_ERR_ARG;
    std::memset(out, 0, sizeof(*out));
    const uint32_t nb = t->numBlocks, P = t->numRowPanels;
    uint32_t *brp = alloc_array<uint32_t>(uint64_t(P) + 1);
    uint64_t *sizePtr = alloc_array<uint64_t>(uint64_t(nb) + 1);
    uint32_t *acols = alloc_array<uint32_t>(uint64_t(nb) * CUTE_TK);
    if (!brp || !sizePtr || !acols) { std::free(brp); std::free(sizePtr); std::free(acols); return CUTE_ERR_NOMEM; }
    std::memcpy(brp, t->blockedRowPtr, (uint64_t(P) + 1) * sizeof(uint32_t));
    for (uint32_t b = 0; b < nb; ++b)
        sizePtr[b + 1] = sizePtr[b] + record_words(t->hdr[uint64_t(b) * CUTE_TILED_HDR_WORDS + 28]);
    uint32_t *stream = alloc_array<uint32_t>(sizePtr[nb]);
    if (!stream) { std::free(brp); std::free(sizePtr); std::free(acols); return CUTE_ERR_NOMEM; }
    uint64_t bricks = 0, nnz = 0;
    for (uint32_t p = 0; p < P; ++p) {
        for (uint32_t b = brp[p]; b < brp[p + 1]; ++b) {
            const uint32_t *hd = t->hdr + uint64_t(b) * CUTE_TILED_HDR_WORDS;
            uint32_t *rec = stream + sizePtr[b];
            uint32_t *ac = acols + uint64_t(b) * CUTE_TK;
            for (uint32_t j = 0; j < 4; ++j)
                for (uint32_t k = 0; k < 4; ++k) ac[j * 4 + k] = hd[k * 4 + j];
            const uint64_t next = sizePtr[b + 1];
            std::memcpy(rec, &next, 8);
            rec[26] = uint32_t((next - sizePtr[b]) / CUTE_CHUNK_WORDS);
            float *dst = reinterpret_cast<float *>(rec + CUTE_META_WORDS);
            uint16_t prefix[4];
            uint64_t col_ptr = 0;
            uint32_t run = 0;
            for (uint32_t j = 0; j < 4; ++j) {
                uint64_t lane;
                std::memcpy(&lane, hd + 16 + 2 * j, 8);
                const uint64_t canon = bitmap_to_canonical(lane);
                std::memcpy(rec + 28 + 2 * j, &canon, 8);
                prefix[j] = uint16_t(run);
                if (canon) { col_ptr |= 1ull << (j * 4); bricks++; }
                rec[4 + j] = uint32_t(__builtin_popcountll(canon & 0xFFFFFFFFull)) |
                             (uint32_t(__builtin_popcountll(canon >> 32)) << 8);
                const float *src = t->vals + hd[24 + j];
                uint64_t rest = canon;
                while (rest) {
                    unsigned cb = unsigned(__builtin_ctzll(rest));
                    rest &= rest - 1;
                    unsigned lb = (cb & 3u) * 16u + (cb >> 2);
                    unsigned lrank = unsigned(__builtin_popcountll(lane & ((1ull << lb) - 1ull)));
                    dst[run++] = src[lrank];
                }
            }
            nnz += run;
            std::memcpy(rec + 24, prefix, 8);
            std::memcpy(rec + 2, &col_ptr, 8);
            if (b > brp[p]) {   // links stored in the previous record of the same panel
                uint32_t *prev = stream + sizePtr[b - 1];
                prev[27] = rec[26];
                // the live column count of a block = number of non-pad columns; pads are
                // zero and so is the default fill, so copying all 16 reproduces both
                std::memcpy(prev + 8, ac, CUTE_TK * sizeof(uint32_t));
            }
        }
    }
    out->M = t->M;
    out->K = t->K;
    out->numRowPanels = P;
    out->numBlocks = nb;
    out->numWords = sizePtr[nb];
    out->blockedRowPtr = brp;
    out->activeCols = acols;
    out->sizePtr = sizePtr;
    out->blocksData = stream;
    out->nnz = uint32_t(nnz);
    out->numBricks = uint32_t(bricks);
    return CUTE_OK;
}

// ---------------------------------------------------------------------------------
// launch partition (spmm.cu:776-812)
// ---------------------------------------------------------------------------------
// The fast kernels (rolling brick kernel, quad kernels) form every B, C and value address as a 32-bit byte
// offset from a scalar base, and the row part of it with a 24 x 24-bit multiply: row index times row pitch.
// That holds while every row and column index and the row pitch in bytes stay below 2^24 and every array
// below 4 GiB -- including the matrix of partial tiles that the pieces of cut panels are stored to, which has
// the row pitch of C and `partial_rows` rows (pieces x rows per piece).
extern "C" int cute_offsets_fit(uint32_t M, uint32_t K, uint32_t N, uint64_t num_vals, uint64_t partial_rows)
{
    const uint64_t lim24 = 1ull << 24, lim32 = 0xffffffffull;
    const uint64_t pitch = uint64_t(N) * 4u;
    return (K < lim24 && uint64_t(M) + 16u < lim24 && pitch < lim24 && uint64_t(K) * pitch <= lim32 &&
            (uint64_t(M) + 16u) * pitch <= lim32 && (num_vals + 64u) * 4u <= lim32 && partial_rows < lim24 &&
            partial_rows * pitch <= lim32)
               ? 1 : 0;
}

extern "C" int64_t cute_partition(uint32_t P, const uint32_t *brp, uint32_t nbN, uint32_t slots,
                                  uint32_t *out4, uint64_t cap)
{
    if (!brp || P == 0 || nbN == 0 || slots == 0) return CUTE_ERR_ARG;
    const uint64_t items = uint64_t(P) * nbN;
    const uint32_t waves = uint32_t((items + slots - 1) / slots);
    const uint32_t avg = std::max<uint32_t>(brp[P] / P, 1u);
    uint64_t n = 0;
    auto emit = [&](uint32_t s, uint32_t e, uint32_t p, uint32_t atomic) {
        if (n < cap && out4) {
            out4[4 * n + 0] = s;
            out4[4 * n + 1] = e;
            out4[4 * n + 2] = p;
            out4[4 * n + 3] = atomic;
        }
        ++n;
    };
    for (uint32_t p = 0; p < P; ++p) {
        const uint32_t s = brp[p], e = brp[p + 1];
        if (s == e) continue;
        const uint32_t nblk = e - s;
        const uint32_t loads = (nblk + avg - 1) / avg;
        const uint32_t ratio = (loads + waves - 1) / waves;
        if (ratio <= 1) { emit(s, e, p, 0); continue; }
        const uint32_t chunk = (nblk + ratio - 1) / ratio;
        for (uint32_t k = 0; k < ratio; ++k) {
            uint32_t cs = s + k * chunk, ce = std::min(e, s + (k + 1) * chunk);
            emit(cs, ce, p, 1);
        }
    }
    return int64_t(n);
}

// ---------------------------------------------------------------------------------
// metrics
// ---------------------------------------------------------------------------------
// CPU SpMM with the sums of inc.h:71-83: C = 0, then every nonzero in array order adds v * B[c,:] onto
// C[r,:], product and sum rounded separately.  The reference forks its thread team inside the loop over
// the nonzeros, once per nonzero; here the nonzeros are first grouped by row (a stable counting sort, so
// each row still sees its nonzeros in array order) and the rows are shared out among the threads, which
// gives every element of C the same sequence of additions, bit for bit, at one fork per call.
#pragma clang fp contract(off)
extern "C" int cute_spmm_coo(const uint32_t *rows, const uint32_t *cols, const float *vals, const float *B, float *C,
                             uint32_t M, uint32_t K, uint32_t N, uint32_t NNZ)
{
    if (!B || !C || (NNZ && (!rows || !cols || !vals))) return CUTE_ERR_ARG;
    if (N == 0) return CUTE_ERR_SHAPE;
    for (uint32_t i = 0; i < NNZ; ++i)
        if (rows[i] >= M || cols[i] >= K) return CUTE_ERR_RANGE;
    std::vector<uint32_t> start(size_t(M) + 1, 0u), order(NNZ);
    for (uint32_t i = 0; i < NNZ; ++i) start[rows[i] + 1]++;
    for (uint32_t r = 0; r < M; ++r) start[r + 1] += start[r];
    {
        std::vector<uint32_t> fill(start.begin(), start.end() - 1);
        for (uint32_t i = 0; i < NNZ; ++i) order[fill[rows[i]]++] = i;
    }
    parallel_ranges(M, 64, [&](uint64_t rb, uint64_t re, unsigned) {
        for (uint64_t r = rb; r < re; ++r) {
            float *c = C + r * N;
            std::memset(c, 0, size_t(N) * sizeof(float));
            for (uint32_t q = start[r]; q < start[r + 1]; ++q) {
                const uint32_t i = order[q];
                const float v = vals[i];
                const float *b = B + size_t(cols[i]) * N;
                for (uint32_t j = 0; j < N; ++j) {
                    const float prod = v * b[j];
                    c[j] += prod;
                }
            }
        }
    });
    return CUTE_OK;
}

extern "C" float cute_check_gemm_correctness(const float *C_ref, const float *C_test, uint32_t M, uint32_t N)
{
    const uint64_t total = uint64_t(M) * N;
    std::vector<float> part(host_threads() + 1, 0.0f);
    parallel_ranges(total, 1 << 16, [&](uint64_t b, uint64_t e, unsigned t) {
        float worst = 0.0f;
        for (uint64_t i = b; i < e; ++i) {
            if (C_ref[i] == 0.0f) continue;                       // inc.h:91-92
            float rel = std::fabs(C_ref[i] - C_test[i]) / std::fabs(C_ref[i]);
            if (rel > worst || rel != rel) worst = rel;           // a NaN result is reported, not hidden
        }
        part[t] = worst;
    });
    float worst = 0.0f;
    for (float x : part)
        if (x > worst || x != x) worst = x;
    return worst;
}

extern "C" float cute_backward_error(const uint32_t *rowPtr, const uint32_t *cols, const float *vals,
                                     const float *B, const float *C_ref, const float *C_test,
                                     uint32_t M, uint32_t N)
{
    std::vector<float> part(host_threads() + 1, 0.0f);
    parallel_ranges(M, 64, [&](uint64_t rb, uint64_t re, unsigned t) {
        std::vector<double> scale(N);
        float worst = 0.0f;
        for (uint64_t r = rb; r < re; ++r) {
            std::fill(scale.begin(), scale.end(), 0.0);
            for (uint32_t i = rowPtr[r]; i < rowPtr[r + 1]; ++i) {
                const float *b = B + uint64_t(cols[i]) * N;
                const double a = std::fabs(double(vals[i]));
                for (uint32_t j = 0; j < N; ++j) scale[j] += a * std::fabs(double(b[j]));
            }
            for (uint32_t j = 0; j < N; ++j) {
                double d = std::fabs(double(C_ref[r * N + j]) - double(C_test[r * N + j]));
                float q = (d == 0.0) ? 0.0f : float(d / scale[j]);   // d>0 with scale 0 -> inf
                if (q > worst || q != q) worst = q;
            }
        }
        part[t] = worst;
    });
    float worst = 0.0f;
    for (float x : part)
        if (x > worst || x != x) worst = x;
    return worst;
}
