// Binary cache of a preprocessed matrix: the CSR arrays plus the four canonical HRPB arrays, so
// that an iterative caller (solver sweeps, training epochs) pays for reading and converting a
// matrix once.  The reference recomputes the format on every run (run.cu:17-20) and has no
// serialisation; the file layout below is this library's own.
//
//   offset  0  char[8]  "CUTEHRPB"
//           8  u32      version (2)
//          12  u32      panel height (16)     16  u32  block width (16)     20  u32  brick width (4)
//          24  u32 M    28 u32 K    32 u32 nnz    36 u32 numRowPanels    40 u32 numBlocks    44 u32 numBricks
//          48  u64      numWords
//          56  u64      FNV-1a 64 of the 56 header bytes before this field, then of every payload byte in file order
//          64  payload: blockedRowPtr[P+1] u32, activeCols[nb*16] u32, sizePtr[nb+1] u64,
//                       blocksData[numWords] u32, rowPtr[M+1] u32, cols[nnz] u32, vals[nnz] f32
// Little-endian, no padding between arrays.  A reader rejects a wrong magic, version, tile shape,
// length or checksum, and -- because a checksum only guards against accidents -- every array whose
// contents could send a later consumer out of bounds: pointers that do not ascend or whose end
// markers disagree with the header, a column or active column >= K, a record offset that is not a
// whole number of 128-word chunks or disagrees with the size the record itself states.
#include "common.hpp"

#include <cstddef>
#include <cstdio>
#include <cstring>

namespace {

constexpr char kMagic[8] = {'C', 'U', 'T', 'E', 'H', 'R', 'P', 'B'};
constexpr uint32_t kVersion = 2;

struct FileHeader {
    char magic[8];
    uint32_t version, tm, tk, brick;
    uint32_t M, K, nnz, numRowPanels, numBlocks, numBricks;
    uint64_t numWords, checksum;
};
static_assert(sizeof(FileHeader) == 64, "header is 64 bytes");

uint64_t fnv1a(uint64_t h, const void *data, uint64_t n)
{
    const unsigned char *p = static_cast<const unsigned char *>(data);
    for (uint64_t i = 0; i < n; ++i) { h ^= p[i]; h *= 0x100000001b3ull; }
    return h;
}

struct Piece { const void *ptr; uint64_t bytes; };

constexpr uint64_t kFnvBasis = 0xcbf29ce484222325ull;
constexpr size_t kHeaderSummed = offsetof(FileHeader, checksum);    // 56: everything in front of the checksum

// What the consumers of a loaded matrix rely on (cute_hrpb_retile walks blocksData by sizePtr, the
// device kernels index B by cols and activeCols, the planner walks rowPtr and blockedRowPtr).
bool arrays_consistent(const FileHeader &fh, const uint32_t *brp, const uint32_t *acols, const uint64_t *sp,
                       const uint32_t *stream, const uint32_t *rp, const uint32_t *cols)
{
    if (brp[0] != 0 || brp[fh.numRowPanels] != fh.numBlocks || sp[0] != 0 || sp[fh.numBlocks] != fh.numWords ||
        rp[0] != 0 || rp[fh.M] != fh.nnz)
        return false;
    for (uint32_t r = 0; r < fh.M; ++r)
        if (rp[r + 1] < rp[r] || rp[r + 1] > fh.nnz) return false;
    for (uint32_t i = 0; i < fh.nnz; ++i)
        if (cols[i] >= fh.K) return false;
    for (uint32_t p = 0; p < fh.numRowPanels; ++p)
        if (brp[p + 1] < brp[p] || brp[p + 1] > fh.numBlocks) return false;
    for (uint64_t i = 0; i < uint64_t(fh.numBlocks) * CUTE_TK; ++i)
        if (acols[i] >= fh.K) return false;
    uint64_t bits = 0, bricks = 0;
    for (uint32_t b = 0; b < fh.numBlocks; ++b) {
        if (sp[b + 1] <= sp[b] || sp[b + 1] > fh.numWords) return false;
        const uint64_t step = sp[b + 1] - sp[b];
        if (step % CUTE_CHUNK_WORDS) return false;
        const uint32_t *rec = stream + sp[b];
        uint32_t nnz_blk = 0;
        for (uint32_t j = 0; j < 4; ++j) {
            uint64_t bm;
            std::memcpy(&bm, rec + 28 + 2 * j, 8);
            nnz_blk += uint32_t(__builtin_popcountll(bm));
            bricks += bm != 0;
        }
        const uint64_t words = (((nnz_blk + 1u) / 2u) * 2u + CUTE_META_WORDS + CUTE_CHUNK_WORDS - 1u) / CUTE_CHUNK_WORDS;
        if (words * CUTE_CHUNK_WORDS != step || rec[26] != words) return false;
        bits += nnz_blk;
    }
    return bits == fh.nnz && bricks == fh.numBricks;
}

}  // namespace

extern "C" {

int cute_hrpb_save(const cute_hrpb_host *h, const char *path)
{
    if (!h || !path || !h->blockedRowPtr || !h->rowPtr) return CUTE_ERR_ARG;
    FileHeader fh{};
    std::memcpy(fh.magic, kMagic, 8);
    fh.version = kVersion;
    fh.tm = CUTE_TM; fh.tk = CUTE_TK; fh.brick = 4;
    fh.M = h->M; fh.K = h->K; fh.nnz = h->nnz;
    fh.numRowPanels = h->numRowPanels; fh.numBlocks = h->numBlocks; fh.numBricks = h->numBricks;
    fh.numWords = h->numWords;
    const Piece pieces[7] = {
        {h->blockedRowPtr, (uint64_t(h->numRowPanels) + 1) * 4}, {h->activeCols, uint64_t(h->numBlocks) * CUTE_TK * 4},
        {h->sizePtr, (uint64_t(h->numBlocks) + 1) * 8},          {h->blocksData, h->numWords * 4},
        {h->rowPtr, (uint64_t(h->M) + 1) * 4},                   {h->cols, uint64_t(h->nnz) * 4},
        {h->vals, uint64_t(h->nnz) * 4}};
    uint64_t sum = fnv1a(kFnvBasis, &fh, kHeaderSummed);
    for (const Piece &p : pieces) sum = fnv1a(sum, p.ptr, p.bytes);
    fh.checksum = sum;
    FILE *f = std::fopen(path, "wb");
    if (!f) return CUTE_ERR_IO;
    bool ok = std::fwrite(&fh, sizeof(fh), 1, f) == 1;
    for (const Piece &p : pieces)
        if (ok && p.bytes) ok = std::fwrite(p.ptr, 1, p.bytes, f) == p.bytes;
    ok = (std::fclose(f) == 0) && ok;
    if (!ok) { std::remove(path); return CUTE_ERR_IO; }
    return CUTE_OK;
}

int cute_hrpb_load(const char *path, cute_csr *csr, cute_hrpb_host *h)
{
    if (!path || !csr || !h) return CUTE_ERR_ARG;
    std::memset(csr, 0, sizeof(*csr));
    std::memset(h, 0, sizeof(*h));
    FILE *f = std::fopen(path, "rb");
    if (!f) return CUTE_ERR_IO;
    FileHeader fh;
    if (std::fread(&fh, sizeof(fh), 1, f) != 1) { std::fclose(f); return CUTE_ERR_FORMAT; }
    if (std::memcmp(fh.magic, kMagic, 8) != 0 || fh.version != kVersion || fh.tm != CUTE_TM || fh.tk != CUTE_TK ||
        fh.brick != 4 || fh.M == 0 || fh.K == 0 || fh.M % CUTE_TM || fh.K % CUTE_TK || fh.numRowPanels != fh.M / CUTE_TM) {
        std::fclose(f);
        return CUTE_ERR_FORMAT;
    }
    const uint64_t bytes[7] = {(uint64_t(fh.numRowPanels) + 1) * 4, uint64_t(fh.numBlocks) * CUTE_TK * 4,
                               (uint64_t(fh.numBlocks) + 1) * 8,    fh.numWords * 4,
                               (uint64_t(fh.M) + 1) * 4,            uint64_t(fh.nnz) * 4, uint64_t(fh.nnz) * 4};
    uint64_t payload = 0;
    for (uint64_t b : bytes) payload += b;
    // the file must hold exactly the payload the header promises (also keeps a forged header
    // from asking for more memory than the file could fill)
    if (std::fseek(f, 0, SEEK_END) != 0 || uint64_t(std::ftell(f)) != sizeof(fh) + payload ||
        std::fseek(f, long(sizeof(fh)), SEEK_SET) != 0) {
        std::fclose(f);
        return CUTE_ERR_FORMAT;
    }
    void *arr[7];
    bool ok = true;
    for (int i = 0; i < 7; ++i) {
        arr[i] = std::malloc(bytes[i] ? bytes[i] : 1);
        ok = ok && arr[i];
    }
    int rc = ok ? CUTE_OK : CUTE_ERR_NOMEM;
    uint64_t sum = fnv1a(kFnvBasis, &fh, kHeaderSummed);
    for (int i = 0; i < 7 && rc == CUTE_OK; ++i) {
        if (bytes[i] && std::fread(arr[i], 1, bytes[i], f) != bytes[i]) rc = CUTE_ERR_FORMAT;
        else sum = fnv1a(sum, arr[i], bytes[i]);
    }
    std::fclose(f);
    if (rc == CUTE_OK && sum != fh.checksum) rc = CUTE_ERR_FORMAT;
    if (rc == CUTE_OK &&
        !arrays_consistent(fh, static_cast<const uint32_t *>(arr[0]), static_cast<const uint32_t *>(arr[1]),
                           static_cast<const uint64_t *>(arr[2]), static_cast<const uint32_t *>(arr[3]),
                           static_cast<const uint32_t *>(arr[4]), static_cast<const uint32_t *>(arr[5])))
        rc = CUTE_ERR_FORMAT;
    if (rc != CUTE_OK) {
        for (void *p : arr) std::free(p);
        return rc;
    }
    csr->M = fh.M; csr->K = fh.K; csr->nnz = fh.nnz;
    csr->rowPtr = static_cast<uint32_t *>(arr[4]);
    csr->cols = static_cast<uint32_t *>(arr[5]);
    csr->vals = static_cast<float *>(arr[6]);
    h->M = fh.M; h->K = fh.K; h->nnz = fh.nnz;
    h->numRowPanels = fh.numRowPanels; h->numBlocks = fh.numBlocks; h->numBricks = fh.numBricks;
    h->numWords = fh.numWords;
    h->blockedRowPtr = static_cast<uint32_t *>(arr[0]);
    h->activeCols = static_cast<uint32_t *>(arr[1]);
    h->sizePtr = static_cast<uint64_t *>(arr[2]);
    h->blocksData = static_cast<uint32_t *>(arr[3]);
    h->rowPtr = csr->rowPtr; h->cols = csr->cols; h->vals = csr->vals;
    return CUTE_OK;
}

}  // extern "C"
