// Walks the host half of the C interface (readers, format builders, cache file, generators, the second API
// family) on small and awkward inputs.  Meant to be compiled together with the library's host sources under
// -fsanitize=address,undefined: the sanitizers do the checking, this program only has to reach the code and
// keeps a few invariants of its own (dense round trips).  No GPU call is made.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "cutespmm.h"

static int g_failures = 0;
#define EXPECT(cond)                                                                  \
    do {                                                                              \
        if (!(cond)) {                                                                \
            std::fprintf(stderr, "line %d: %s\n", __LINE__, #cond);                   \
            ++g_failures;                                                             \
        }                                                                             \
    } while (0)

static const uint64_t kDenseLimit = 1u << 20;

static std::vector<float> dense_of_csr(const cute_csr &a)
{
    std::vector<float> d(size_t(a.M) * a.K, 0.0f);
    for (uint32_t r = 0; r < a.M; ++r)
        for (uint32_t i = a.rowPtr[r]; i < a.rowPtr[r + 1]; ++i) d[size_t(r) * a.K + a.cols[i]] += a.vals[i];
    return d;
}

// Decodes the device layout of the brick kernel (header lines + values in lane order) back to a dense matrix.
static std::vector<float> dense_of_tiled(const cute_hrpb_tiled &t)
{
    std::vector<float> d(size_t(t.M) * t.K, 0.0f);
    for (uint32_t q = 0; q < t.numRowPanels; ++q)
        for (uint32_t b = t.blockedRowPtr[q]; b < t.blockedRowPtr[q + 1]; ++b) {
            const uint32_t *h = t.hdr + size_t(b) * 32;
            for (int j = 0; j < 4; ++j) {
                const uint64_t bits = uint64_t(h[16 + 2 * j]) | (uint64_t(h[17 + 2 * j]) << 32);
                uint32_t at = h[24 + j];
                for (int lane = 0; lane < 64; ++lane)
                    if (bits >> lane & 1) {
                        const int k = lane / 16, row = lane % 16;
                        d[size_t(q * 16 + row) * t.K + h[k * 4 + j]] += t.vals[at++];
                    }
            }
        }
    return d;
}

static std::vector<float> dense_of_quad(const cute_quad_lists &ql)
{
    std::vector<float> d(size_t(ql.M) * ql.K, 0.0f);
    for (uint32_t u = 0; u < ql.numRowPanels; ++u)
        for (uint32_t g = ql.groupPtr[u]; g < ql.groupPtr[u + 1]; ++g)
            for (int p = 0; p < 16; ++p) {
                const uint32_t col = ql.cols[size_t(g) * 16 + p];
                const uint32_t row0 = ql.rowsPerList == 16 ? u * 16 + 4 * (p % 4) : u * 4;
                for (int i = 0; i < 4; ++i) {
                    const float v = ql.vals[size_t(g) * 64 + 4 * p + i];
                    if (v != 0.0f && row0 + i < ql.M) d[size_t(row0 + i) * ql.K + col] += v;
                }
            }
    return d;
}

static void walk_unsigned_family(const cute_csr &a, const std::string &tmp)
{
    const bool small = uint64_t(a.M) * a.K <= kDenseLimit;          // dense round trips on small matrices only
    const std::vector<float> want = small ? dense_of_csr(a) : std::vector<float>();
    cute_hrpb_host h{};
    EXPECT(cute_hrpb_build(a.M, a.K, a.rowPtr, a.cols, a.vals, &h) == CUTE_OK);
    EXPECT(h.numRowPanels == a.M / 16 && h.nnz == a.nnz);

    cute_hrpb_tiled t{};
    EXPECT(cute_hrpb_retile(&h, &t) == CUTE_OK);
    if (small) EXPECT(dense_of_tiled(t) == want);
    cute_hrpb_host back{};
    EXPECT(cute_hrpb_untile(&t, &back) == CUTE_OK);
    EXPECT(back.numWords == h.numWords && back.numBlocks == h.numBlocks);
    if (back.numWords == h.numWords) EXPECT(std::memcmp(back.blocksData, h.blocksData, h.numWords * 4) == 0);
    cute_hrpb_host_release(&back);
    cute_hrpb_tiled_release(&t);

    for (uint32_t slots : {1u, 7u, 2048u, 8192u}) {
        std::vector<uint32_t> quads(4 * (size_t(h.numRowPanels) + slots + 8));
        const int64_t n = cute_partition(h.numRowPanels, h.blockedRowPtr, 2, slots, quads.data(), quads.size() / 4);
        EXPECT(n >= 0 && uint64_t(n) <= quads.size() / 4);
        uint64_t covered = 0;
        for (int64_t i = 0; i < n && uint64_t(i) < quads.size() / 4; ++i) covered += quads[4 * i + 1] - quads[4 * i];
        EXPECT(covered == h.numBlocks);
    }

    cute_quad_lists ql{};
    EXPECT(cute_quad_build(a.M, a.K, a.rowPtr, a.cols, a.vals, &ql) == CUTE_OK);
    if (small) EXPECT(dense_of_quad(ql) == want);
    uint64_t groups = 0, pairs = 0;
    EXPECT(cute_quad_fill(a.M, a.rowPtr, a.cols, &groups, &pairs) == CUTE_OK);
    EXPECT(groups == ql.numGroups);
    cute_quad_release(&ql);
    EXPECT(cute_quad_build_strips(a.M, a.K, a.rowPtr, a.cols, a.vals, &ql) == CUTE_OK);
    if (small) EXPECT(dense_of_quad(ql) == want);
    cute_quad_release(&ql);

    // the device form of the lists, written from the census
    const uint32_t strips = (a.M + 3) / 4;
    std::vector<uint32_t> stripPairs(strips), stripVals(strips);
    EXPECT(cute_quad_census(a.M, a.rowPtr, a.cols, a.vals, stripPairs.data(), stripVals.data()) == CUTE_OK);
    {
        std::vector<uint32_t> groupPtr(strips + 1, 0);
        std::vector<uint64_t> valBase(strips, 0);
        uint64_t vals = 0;
        for (uint32_t s = 0; s < strips; ++s) {
            groupPtr[s + 1] = groupPtr[s] + (stripPairs[s] + 15) / 16;
            valBase[s] = vals;
            vals += stripVals[s];
        }
        std::vector<uint32_t> recs(size_t(groupPtr[strips]) * CUTE_QUAD_RECORD_WORDS + 1);
        std::vector<float> packed(vals + 1);
        EXPECT(cute_quad_pack(a.M, a.rowPtr, a.cols, a.vals, 4, groupPtr.data(), valBase.data(), recs.data(), packed.data()) == CUTE_OK);
    }

    if (!tmp.empty()) {       // cache file: round trip, then damaged copies must be refused, never read out of bounds
        const std::string path = tmp + "/walk.hrpb";
        EXPECT(cute_hrpb_save(&h, path.c_str()) == CUTE_OK);
        cute_csr csr2{};
        cute_hrpb_host h2{};
        EXPECT(cute_hrpb_load(path.c_str(), &csr2, &h2) == CUTE_OK);
        EXPECT(h2.numWords == h.numWords && csr2.nnz == a.nnz);
        cute_hrpb_host_release(&h2);
        cute_csr_release(&csr2);
        std::vector<unsigned char> bytes;
        if (FILE *f = std::fopen(path.c_str(), "rb")) {
            unsigned char buf[4096];
            size_t got;
            while ((got = std::fread(buf, 1, sizeof buf, f)) > 0) bytes.insert(bytes.end(), buf, buf + got);
            std::fclose(f);
        }
        const std::string bad = tmp + "/bad.hrpb";
        for (int variant = 0; variant < 6 && bytes.size() > 64; ++variant) {
            std::vector<unsigned char> b = bytes;
            if (variant == 0) b.resize(b.size() / 2);
            else if (variant == 1) b.resize(17);
            else if (variant == 2) b[b.size() / 2] ^= 0x40;
            else if (variant == 3) for (int i = 8; i < 40; ++i) b[i] = 0xff;       // sizes in the header
            else if (variant == 4) b.insert(b.end(), 64, 0);
            else b[b.size() - 1] ^= 1;
            if (FILE *f = std::fopen(bad.c_str(), "wb")) {
                std::fwrite(b.data(), 1, b.size(), f);
                std::fclose(f);
            }
            cute_csr c3{};
            cute_hrpb_host h3{};
            EXPECT(cute_hrpb_load(bad.c_str(), &c3, &h3) != CUTE_OK);
        }
    }
    cute_hrpb_host_release(&h);

    // CPU SpMM and the two error measures
    const uint32_t N = 8;
    std::vector<float> B(size_t(a.K) * N), C(size_t(a.M) * N), C2;
    cute_gen_dense(3, 1, B.size(), B.data());
    std::vector<uint32_t> rows(a.nnz);
    for (uint32_t r = 0; r < a.M; ++r)
        for (uint32_t i = a.rowPtr[r]; i < a.rowPtr[r + 1]; ++i) rows[i] = r;
    EXPECT(cute_spmm_coo(rows.data(), a.cols, a.vals, B.data(), C.data(), a.M, a.K, N, a.nnz) == CUTE_OK);
    C2 = C;
    EXPECT(cute_check_gemm_correctness(C.data(), C2.data(), a.M, N) == 0.0f);
    EXPECT(cute_backward_error(a.rowPtr, a.cols, a.vals, B.data(), C.data(), C2.data(), a.M, N) == 0.0f);
}

static void walk_signed_family(const cute_csr &a, const std::string &tmp)
{
    cute_coo coo{};
    coo.dimY = int32_t(a.M);
    coo.dimX = int32_t(a.K);
    coo.nnz = int32_t(a.nnz);
    coo.rows = static_cast<int32_t *>(std::malloc(sizeof(int32_t) * (a.nnz + 1)));
    coo.cols = static_cast<int32_t *>(std::malloc(sizeof(int32_t) * (a.nnz + 1)));
    coo.values = static_cast<float *>(std::malloc(sizeof(float) * (a.nnz + 1)));
    for (uint32_t r = 0; r < a.M; ++r)
        for (uint32_t i = a.rowPtr[r]; i < a.rowPtr[r + 1]; ++i) {
            coo.rows[i] = int32_t(r);
            coo.cols[i] = int32_t(a.cols[i]);
            coo.values[i] = a.vals[i];
        }
    cute_csr_i32 csr{};
    EXPECT(cute_coo_to_csr(&coo, &csr) == CUTE_OK);
    EXPECT(csr.nnz == coo.nnz && csr.nrows == coo.dimY);
    if (!tmp.empty() && coo.nnz > 0) {       // (an empty matrix is saved as an empty file, SparseCoo.hpp:275-283)
        const std::string path = tmp + "/walk.mtx";
        EXPECT(cute_coo_save_mtx(&coo, path.c_str()) == CUTE_OK);
        cute_coo again{};
        const int st = cute_coo_read(path.c_str(), &again);
        if (st != CUTE_OK) std::fprintf(stderr, "reading back %d x %d with %d entries: %s\n", coo.dimY, coo.dimX, coo.nnz, cute_status_string(st));
        EXPECT(st == CUTE_OK);
        EXPECT(again.nnz == coo.nnz && again.dimY == coo.dimY && again.dimX == coo.dimX);
        EXPECT(cute_coo_merge_duplicates(&again) == CUTE_OK);
        cute_coo_release(&again);
    }
    std::free(coo.rows);
    std::free(coo.cols);
    std::free(coo.values);

    const bool small = uint64_t(a.M) * a.K <= kDenseLimit;
    std::vector<float> dense(small ? size_t(csr.nrows) * csr.ncols : 0, 0.0f);
    if (small) {
        EXPECT(cute_csr_to_dense(&csr, dense.data()) == CUTE_OK);
        EXPECT(dense == dense_of_csr(a));
    }

    for (int bs : {16, 32}) {
        if (csr.nrows % bs || csr.ncols % bs) continue;
        cute_blocked_ell ell{};
        EXPECT(cute_blocked_ell_build(&csr, bs, &ell) == CUTE_OK);
        if (small) {
            std::vector<float> d2(size_t(ell.height) * bs * csr.ncols, 0.0f);
            EXPECT(cute_blocked_ell_to_dense(&ell, csr.ncols, d2.data()) == CUTE_OK);
            EXPECT(d2.size() >= dense.size() && std::equal(dense.begin(), dense.end(), d2.begin()));
        }
        cute_blocked_ell_release(&ell);

        EXPECT(cute_csr_count_blocks(&csr, bs, 4) >= 0);
        cute_bcsr bc{};
        EXPECT(cute_csr_to_bcsr(&csr, bs, 4, &bc) == CUTE_OK);
        EXPECT(bc.nblks == cute_csr_count_blocks(&csr, bs, 4));
        cute_bcsr_release(&bc);

        for (int thr : {1, 8, bs * bs}) {
            cute_split sp{};
            EXPECT(cute_splitter_split(&csr, bs, thr, &sp) == CUTE_OK);
            EXPECT(sp.numHeavyElems + sp.numLightElems == csr.nnz && sp.numHeavyTiles + sp.numLightTiles == sp.totalTiles);
            cute_split_release(&sp);
        }
        cute_block_class *cls = nullptr;
        int64_t count = 0;
        EXPECT(cute_classify_blocks(&csr, bs, 0.5f, 0.5f, &cls, &count) == CUTE_OK);
        int64_t entries = 0;
        for (int64_t i = 0; i < count; ++i) entries += cls[i].nnz;
        EXPECT(entries == csr.nnz);
        cute_free(cls);
        cute_split sp{};
        EXPECT(cute_split_by_class(&csr, bs, 0.5f, 0.5f, &sp) == CUTE_OK);
        EXPECT(sp.numHeavyElems + sp.numLightElems == csr.nnz);
        cute_split_release(&sp);
        float stats[4], anxs = 0.0f;
        EXPECT(cute_block_stats(&csr, bs, stats) == CUTE_OK);
        EXPECT(cute_anxs(&csr, bs, 1, &anxs) == CUTE_OK);
        EXPECT(cute_anxs(&csr, bs, 0, &anxs) == CUTE_OK);
    }

    const int32_t n = 4;
    std::vector<double> v64(size_t(csr.nnz) + 1), B(size_t(csr.ncols) * n, 0.5), C(size_t(csr.nrows) * n, 0.0);
    for (int32_t i = 0; i < csr.nnz; ++i) v64[i] = csr.values[i];
    EXPECT(cute_sequential_spmm(&csr, v64.data(), B.data(), C.data(), csr.nrows, csr.ncols, n) >= 0.0f);
    cute_csr_i32_release(&csr);
}

static void write_text(const std::string &path, const char *text)
{
    if (FILE *f = std::fopen(path.c_str(), "w")) {
        std::fputs(text, f);
        std::fclose(f);
    }
}

int main(int argc, char **argv)
{
    if (argc < 3) return 2;
    const std::string golden = argv[1], tmp = argv[2];

    // the reference's own matrix through both readers
    for (int keep = 0; keep < 2; ++keep) {
        cute_csr a{};
        EXPECT(cute_mtx_read(golden.c_str(), keep, &a) == CUTE_OK);
        EXPECT(cute_csr_sort_rows(&a) == CUTE_OK || true);
        walk_unsigned_family(a, keep ? tmp : std::string());
        if (keep) walk_signed_family(a, tmp);
        cute_csr_release(&a);
    }
    {
        cute_coo coo{};
        EXPECT(cute_coo_read(golden.c_str(), &coo) == CUTE_OK);
        cute_coo_release(&coo);
    }

    // generated matrices: every kind, with sizes that leave ragged last panels' worth of structure
    struct { int kind; uint32_t p0, p1, p2; } gens[] = {
        {1, 64, 5, 0}, {1, 16, 16, 0}, {2, 8, 0, 0}, {2, 12, 0, 0}, {3, 16, 8, 0}, {4, 6, 4, 0}, {5, 96, 7, 20}, {5, 48, 1, 0},
    };
    for (const auto &g : gens) {
        cute_csr a{};
        const int st = cute_gen_matrix(g.kind, 11, g.p0, g.p1, g.p2, &a);
        if (st != CUTE_OK) std::fprintf(stderr, "generator %d (%u, %u, %u): %s\n", g.kind, g.p0, g.p1, g.p2, cute_status_string(st));
        EXPECT(st == CUTE_OK);
        if (st == CUTE_OK && a.M % 16 == 0 && a.K % 16 == 0) {
            walk_unsigned_family(a, tmp);
            walk_signed_family(a, tmp);
        }
        cute_csr_release(&a);
    }
    {
        cute_csr a{};
        EXPECT(cute_gen_matrix(9, 1, 16, 1, 1, &a) != CUTE_OK);
        EXPECT(cute_gen_matrix(1, 1, 16, 17, 0, &a) != CUTE_OK || a.nnz > 0);
        cute_csr_release(&a);
        float x[5];
        for (int dist = 0; dist < 3; ++dist) EXPECT(cute_gen_dense(5, dist, 5, x) == CUTE_OK);
        EXPECT(cute_gen_dense(5, 7, 5, x) != CUTE_OK);
    }

    // hand-made shapes: empty matrix, one entry, one full row, one full column, a dense panel
    {
        const uint32_t M = 32, K = 48;
        std::vector<std::vector<uint32_t>> shapes_rows[5];
        auto run = [&](const std::vector<std::vector<uint32_t>> &rows) {
            cute_csr a{};
            a.M = M;
            a.K = K;
            std::vector<uint32_t> rp(M + 1, 0), cl;
            std::vector<float> vl;
            for (uint32_t r = 0; r < M; ++r) {
                for (uint32_t c : rows[r]) {
                    cl.push_back(c);
                    vl.push_back(float(r + 1) - 0.25f * float(c));
                }
                rp[r + 1] = uint32_t(cl.size());
            }
            cl.push_back(0);
            vl.push_back(0.0f);
            a.nnz = rp[M];
            a.rowPtr = rp.data();
            a.cols = cl.data();
            a.vals = vl.data();
            walk_unsigned_family(a, tmp);
            walk_signed_family(a, tmp);
        };
        std::vector<std::vector<uint32_t>> rows(M);
        run(rows);                                        // empty
        rows[31] = {47};
        run(rows);                                        // one entry in the last corner
        rows.assign(M, {});
        for (uint32_t c = 0; c < K; ++c) rows[5].push_back(c);
        run(rows);                                        // one full row
        rows.assign(M, {});
        for (uint32_t r = 0; r < M; ++r) rows[r] = {17};
        run(rows);                                        // one full column
        rows.assign(M, {});
        for (uint32_t r = 16; r < 32; ++r)
            for (uint32_t c = 0; c < K; ++c) rows[r].push_back(c);
        run(rows);                                        // a dense panel under an empty one
    }

    // precondition failures come back as statuses
    {
        uint32_t rp[17] = {0}, cl[2] = {3, 3};
        float vl[2] = {1.0f, 2.0f};
        for (int r = 1; r <= 16; ++r) rp[r] = 2;
        cute_hrpb_host h{};
        EXPECT(cute_hrpb_build(16, 16, rp, cl, vl, &h) != CUTE_OK);       // duplicate column
        EXPECT(cute_hrpb_build(15, 16, rp, cl, vl, &h) != CUTE_OK);       // M not a multiple of 16
        cl[1] = 16;
        EXPECT(cute_hrpb_build(16, 16, rp, cl, vl, &h) != CUTE_OK);       // column out of range
        EXPECT(cute_hrpb_build(16, 16, nullptr, cl, vl, &h) != CUTE_OK);
        cute_csr a{};
        a.M = 16, a.K = 16, a.nnz = 2, a.rowPtr = rp, a.cols = cl, a.vals = vl;
        cl[0] = 3, cl[1] = 3;
        EXPECT(cute_csr_sort_rows(&a) == CUTE_ERR_UNSORTED);
    }

    // malformed MatrixMarket files: a status, never a crash
    const char *texts[] = {
        "",
        "%%MatrixMarket matrix coordinate real general\n",
        "%%MatrixMarket matrix coordinate real general\n3 3\n",
        "%%MatrixMarket matrix coordinate real general\n3 3 2\n1 1 1.0\n",
        "%%MatrixMarket matrix coordinate real general\n3 3 1\n4 1 1.0\n",
        "%%MatrixMarket matrix coordinate real general\n3 3 1\n0 1 1.0\n",
        "%%MatrixMarket matrix coordinate real general\n3 3 1\n1 -1 1.0\n",
        "%%MatrixMarket matrix coordinate complex general\n3 3 1\n1 1 1.0 2.0\n",
        "%%MatrixMarket matrix coordinate real hermitian\n3 3 1\n1 1 1.0\n",
        "%%MatrixMarket matrix array real general\n2 2\n1.0\n2.0\n3.0\n",
        "%%MatrixMarket matrix coordinate real general\n4000000000 4000000000 1\n1 1 1.0\n",
        "%%MatrixMarket matrix coordinate real general\n3 3 99999999999\n1 1 1.0\n",
        "%%MatrixMarket matrix coordinate real general\n3 3 1\n1 1 notanumber\n",
        "%%MatrixMarket matrix coordinate pattern symmetric\n3 3 2\n2 1\n3 3\n",
        "%%MatrixMarket matrix coordinate real skew-symmetric\n3 3 1\n2 1 5.0\n",
        "%%MatrixMarket matrix array real general\n2 2\n1.0\n0.0\n0.0\n4.0\n",
        "3 3 1\n1 1 1.0\n",
    };
    int accepted = 0;
    for (size_t i = 0; i < sizeof texts / sizeof texts[0]; ++i) {
        const std::string path = tmp + "/m" + std::to_string(i) + ".mtx";
        write_text(path, texts[i]);
        for (int keep = 0; keep < 2; ++keep) {
            cute_csr a{};
            if (cute_mtx_read(path.c_str(), keep, &a) == CUTE_OK) {
                ++accepted;
                EXPECT(a.M % 16 == 0 && a.K % 16 == 0 && a.rowPtr[a.M] == a.nnz);
                for (uint32_t e = 0; e < a.nnz; ++e) EXPECT(a.cols[e] < a.K);
                cute_csr_release(&a);
            }
        }
        cute_coo coo{};
        if (cute_coo_read(path.c_str(), &coo) == CUTE_OK) {
            for (int32_t e = 0; e < coo.nnz; ++e) EXPECT(coo.rows[e] >= 0 && coo.rows[e] < coo.dimY && coo.cols[e] >= 0 && coo.cols[e] < coo.dimX);
            cute_coo_release(&coo);
        }
    }
    EXPECT(accepted >= 4);          // the last four are well-formed for at least one reader

    EXPECT(std::strlen(cute_status_string(CUTE_ERR_FORMAT)) > 0 && std::strlen(cute_status_string(12345)) > 0);
    std::printf("host sanitize walk: %d failures\n", g_failures);
    return g_failures ? 1 : 0;
}
