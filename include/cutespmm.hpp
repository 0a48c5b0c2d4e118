// cutespmm.hpp -- the reference's C++ host classes, re-stated over the C ABI of libcutespmm.
//
// Same class names, public fields and call sequence as the reference's driver uses
// (run.cu:11-62):   MTX_READER r(path);  HRPB hrpb(M, K, r.rowPtr, r.cols, r.vals);
//                   SPMM_TC spmm(M, K, N, hrpb.blockedRowPtr);
//                   spmm.run(hrpb.blocksDevice, dB, dC, hrpb.activeColsDevice, hrpb.sizePtrDevice);
// (or the shorter forms SPMM_TC spmm(M, K, N, hrpb); spmm.run(dB, dC, stream);).
// Differences, all deliberate: every object frees what it owns; errors throw
// cute::Error instead of exit(-1) (inc.h:63-70) or a float-typed EXIT_FAILURE
// (spmm.cu:841-859); HRPB checks its preconditions; C need not be zeroed by the caller.
#pragma once
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>

#include "cutespmm.h"

namespace cute {

struct Error : std::runtime_error {
    int status;
    Error(int s, const std::string &where)
        : std::runtime_error(where + ": " + cute_status_string(s) +
                             ((s == CUTE_ERR_HIP || s == CUTE_ERR_NO_DEVICE) ? std::string(" -- ") + cute_last_hip_error() : "")),
          status(s) {}
};
inline void check(int s, const char *where) { if (s != CUTE_OK) throw Error(s, where); }

// The reference's planner is constructed from the format's blockedRowPtr array alone (spmm.cu:276) and its
// run() is handed three more device arrays of the same format (spmm.cu:823).  Here the device side of a
// format is one handle, so every live HRPB is listed under the address of its blockedRowPtr array and the
// reference-shaped SPMM_TC constructor finds the format -- and with it the handle -- from that pointer.
struct HrpbRegistry {
    std::mutex lock;
    std::map<const unsigned int *, const void *> live;     // blockedRowPtr -> HRPB object
    static HrpbRegistry &get() { static HrpbRegistry r; return r; }
};

}  // namespace cute

// IO.cu:2-88
class MTX_READER {
public:
    unsigned int M = 0, K = 0, nnz = 0;
    unsigned int *rowPtr = nullptr;
    unsigned int *cols = nullptr;
    float *vals = nullptr;
    explicit MTX_READER(const std::string &file_path, bool keep_values = false)
    {
        cute::check(cute_mtx_read(file_path.c_str(), keep_values ? 1 : 0, &csr_), "MTX_READER");
        adopt();
    }
    // Wraps a generated matrix (cute_gen_matrix) in the same fields.
    explicit MTX_READER(const cute_csr &owned) : csr_(owned) { adopt(); }
    void sort_rows() { cute::check(cute_csr_sort_rows(&csr_), "MTX_READER::sort_rows"); }
    ~MTX_READER() { cute_csr_release(&csr_); }
    MTX_READER(const MTX_READER &) = delete;
    MTX_READER &operator=(const MTX_READER &) = delete;

private:
    cute_csr csr_{};
    void adopt() { M = csr_.M; K = csr_.K; nnz = csr_.nnz; rowPtr = csr_.rowPtr; cols = csr_.cols; vals = csr_.vals; }
};

// data.cu:54-340
class HRPB {
public:
    unsigned int *cols, *rowPtr;      // borrowed, as in data.cu:82-84
    float *vals;
    unsigned int M, K, numRowPanels;
    unsigned int *blocksData = nullptr;
    unsigned long long dataStructSize = 0;
    unsigned int num_bricks = 0;
    unsigned int *blockedRowPtr = nullptr;
    unsigned long long *sizePtr = nullptr;
    unsigned int *activeCols = nullptr;
    unsigned int numNNZ = 0;
    float block_density = 0.0f;       // nonzeros per slot of the non-empty bricks
    cute_hrpb_dev *device = nullptr;  // the device copy (both MFMA layouts and the CSR arrays)
    // The four *Device fields of data.cu:65-72.  The device copy is not the canonical stream, so these are
    // not addresses of such arrays: they are tokens (the handle above, retyped; null without a device copy)
    // whose only use is to be passed to SPMM_TC::run as run.cu:46-50 does, which checks them.
    unsigned int *blocksDevice = nullptr, *blockedRowPtrDevice = nullptr, *activeColsDevice = nullptr;
    unsigned long long *sizePtrDevice = nullptr;

    HRPB(unsigned int M_, unsigned int K_, unsigned int *rowPtr_, unsigned int *cols_, float *vals_, bool upload = true)
        : cols(cols_), rowPtr(rowPtr_), vals(vals_), M(M_), K(K_), numRowPanels(M_ / CUTE_TM)
    {
        cute::check(cute_hrpb_build(M, K, rowPtr, cols, vals, &host_), "HRPB");
        publish(upload);
    }
    // Reads what save() wrote (no counterpart in the reference, which rebuilds the format on every
    // run): the object then owns its CSR arrays as well.
    explicit HRPB(const char *cache_file, bool upload = true)
    {
        cute::check(cute_hrpb_load(cache_file, &owned_csr_, &host_), "HRPB cache file");
        cols = owned_csr_.cols; rowPtr = owned_csr_.rowPtr; vals = owned_csr_.vals;
        M = host_.M; K = host_.K; numRowPanels = host_.numRowPanels;
        publish(upload);
    }
    void save(const char *cache_file) const { cute::check(cute_hrpb_save(&host_, cache_file), "HRPB save"); }
    void freeDevice()                                                       // data.cu:336-339
    {
        cute_hrpb_dev_free(device);
        device = nullptr;
        blocksDevice = blockedRowPtrDevice = activeColsDevice = nullptr;
        sizePtrDevice = nullptr;
    }
    const cute_hrpb_host &host() const { return host_; }
    // The live format whose blockedRowPtr array this is, or null.
    static const HRPB *find(const unsigned int *blockedRowPtr_)
    {
        cute::HrpbRegistry &r = cute::HrpbRegistry::get();
        std::lock_guard<std::mutex> g(r.lock);
        auto it = r.live.find(blockedRowPtr_);
        return it == r.live.end() ? nullptr : static_cast<const HRPB *>(it->second);
    }
    ~HRPB()
    {
        {
            cute::HrpbRegistry &r = cute::HrpbRegistry::get();
            std::lock_guard<std::mutex> g(r.lock);
            r.live.erase(blockedRowPtr);
        }
        freeDevice();
        cute_hrpb_host_release(&host_);
        cute_csr_release(&owned_csr_);
    }
    HRPB(const HRPB &) = delete;
    HRPB &operator=(const HRPB &) = delete;

private:
    cute_hrpb_host host_{};
    cute_csr owned_csr_{};
    void publish(bool upload)
    {
        blocksData = host_.blocksData;
        dataStructSize = host_.numWords;
        num_bricks = host_.numBricks;
        blockedRowPtr = host_.blockedRowPtr;
        sizePtr = reinterpret_cast<unsigned long long *>(host_.sizePtr);
        activeCols = host_.activeCols;
        numNNZ = host_.nnz;
        block_density = num_bricks ? float(numNNZ) / (64.0f * float(num_bricks)) : 0.0f;
        if (upload) {
            int rc = cute_hrpb_upload(&host_, &device);
            if (rc != CUTE_OK) { cute_hrpb_host_release(&host_); cute_csr_release(&owned_csr_); throw cute::Error(rc, "HRPB upload"); }
            blocksDevice = blockedRowPtrDevice = activeColsDevice = reinterpret_cast<unsigned int *>(device);
            sizePtrDevice = reinterpret_cast<unsigned long long *>(device);
        }
        cute::HrpbRegistry &r = cute::HrpbRegistry::get();
        std::lock_guard<std::mutex> g(r.lock);
        r.live[blockedRowPtr] = this;
    }
};

// The format built on the device from CSR arrays that already live there (device pointers): what the HRPB
// constructor does on the host (data.cu:80-335), by kernels.  It has no canonical host arrays to inspect; it
// takes the place of an HRPB in SPMM_TC(M, K, N, hrpb).
class HRPB_DEVICE {
public:
    unsigned int M, K, numNNZ;
    cute_hrpb_dev *device = nullptr;
    HRPB_DEVICE(unsigned int M_, unsigned int K_, unsigned int nnz, const unsigned int *rowPtrDevice, const unsigned int *colsDevice,
                const float *valsDevice, int quad_layout = 0)
        : M(M_), K(K_), numNNZ(nnz)
    {
        cute::check(cute_hrpb_upload_device_csr(M, K, nnz, rowPtrDevice, colsDevice, valsDevice, quad_layout, &device), "HRPB_DEVICE");
    }
    ~HRPB_DEVICE() { cute_hrpb_dev_free(device); }
    HRPB_DEVICE(const HRPB_DEVICE &) = delete;
    HRPB_DEVICE &operator=(const HRPB_DEVICE &) = delete;
};

// spmm.cu:258-840
class SPMM_TC {
public:
    unsigned int M, N, K;
    unsigned int numRowPanelsSplit = 0;
    cute_plan_info info{};
    SPMM_TC(unsigned int M_, unsigned int K_, unsigned int N_, const HRPB &hrpb, const cute_tunables *tunables = nullptr)
        : M(M_), N(N_), K(K_)
    {
        create(hrpb, tunables);
    }
    SPMM_TC(unsigned int M_, unsigned int K_, unsigned int N_, const HRPB_DEVICE &hrpb, const cute_tunables *tunables = nullptr)
        : M(M_), N(N_), K(K_)
    {
        create(hrpb.device, tunables);
    }
    // The reference's own signature (spmm.cu:276; call site run.cu:45): the format is found from its
    // blockedRowPtr array, which must belong to a live HRPB object that has a device copy.
    SPMM_TC(unsigned int M_, unsigned int K_, unsigned int N_, unsigned int *blockedRowPtr) : M(M_), N(N_), K(K_)
    {
        const HRPB *hrpb = HRPB::find(blockedRowPtr);
        if (!hrpb) throw cute::Error(CUTE_ERR_ARG, "SPMM_TC: blockedRowPtr does not belong to a live HRPB");
        if (hrpb->M != M || hrpb->K != K) throw cute::Error(CUTE_ERR_SHAPE, "SPMM_TC: M, K differ from the HRPB's");
        create(*hrpb, nullptr);
    }
    // MatB [K x N], MatC [M x N]: device pointers; asynchronous on `stream`.
    void run(const float *MatB, float *MatC, void *stream = nullptr)
    {
        cute::check(cute_spmm_run(plan_, MatB, MatC, stream), "SPMM_TC::run");
    }
    // The reference's own signature (spmm.cu:823; call site run.cu:50), asynchronous on the default stream.
    // The three format arguments must be the *Device fields of the HRPB this plan was made for; the plan
    // already holds that format, so they are only checked.
    void run(unsigned int *MatA, float *MatB, float *MatC, unsigned int *active_cols_vec, unsigned long long int *sizePtr)
    {
        const void *want = format_;
        if (MatA != want || active_cols_vec != want || sizePtr != want)
            throw cute::Error(CUTE_ERR_ARG, "SPMM_TC::run: MatA, active_cols_vec, sizePtr are not this plan's HRPB device fields");
        run(MatB, MatC, nullptr);
    }
    // With the partial tiles of cut panels in the caller's buffer (scratch_bytes() bytes of device memory):
    // one plan can then run on several streams at once.
    uint64_t scratch_bytes() const { return cute_spmm_plan_scratch_bytes(plan_); }
    void run(const float *MatB, float *MatC, void *stream, void *scratch, uint64_t bytes)
    {
        cute::check(cute_spmm_run_scratch(plan_, MatB, MatC, stream, scratch, bytes), "SPMM_TC::run");
    }
    cute_spmm_plan *plan() { return plan_; }
    ~SPMM_TC() { cute_spmm_plan_free(plan_); }
    SPMM_TC(const SPMM_TC &) = delete;
    SPMM_TC &operator=(const SPMM_TC &) = delete;

private:
    cute_spmm_plan *plan_ = nullptr;
    const cute_hrpb_dev *format_ = nullptr;
    void create(const HRPB &hrpb, const cute_tunables *tunables) { create(hrpb.device, tunables); }
    void create(cute_hrpb_dev *device, const cute_tunables *tunables)
    {
        if (!device) throw cute::Error(CUTE_ERR_ARG, "SPMM_TC: HRPB has no device copy");
        cute::check(cute_spmm_plan_create(device, N, tunables, &plan_), "SPMM_TC");
        cute_spmm_plan_info(plan_, &info);
        numRowPanelsSplit = info.numChunks;
        format_ = device;
    }
};

// inc.h:71-83
inline void spmm_coo(unsigned int *rows, unsigned int *cols, float *vals, float *B, float *C, uint32_t M, uint32_t K,
                     uint32_t N, unsigned int NNZ)
{
    cute::check(cute_spmm_coo(rows, cols, vals, B, C, M, K, N, NNZ), "spmm_coo");
}

// inc.h:84-109
inline float check_gemm_correctness_coo(float *C, float *C_HOST, uint32_t M, uint32_t N)
{
    return cute_check_gemm_correctness(C, C_HOST, M, N);
}

// spmm.cu:860-861 (host arrays in, host C out, ms per launch; alpha = 1, beta = 0 only)
inline float GPU_CSR_cuSPARSE_NEW(unsigned int *hA_csrOffsets, unsigned int *hA_columns, float *hA_values,
                                  unsigned int A_nnz, float *hB, float *hC, uint32_t m, uint32_t k, uint32_t n, int iters)
{
    float ms = cute_gpu_csr_spmm(hA_csrOffsets, hA_columns, hA_values, A_nnz, hB, hC, m, k, n, iters, 2);
    if (ms < 0) throw cute::Error(int(ms), "GPU_CSR_cuSPARSE_NEW");
    return ms;
}

// ---------------------------------------------------------------------------------------
// Second API family (inc/SparseCoo.hpp, inc/CSR.hpp, inc/prepareBlkEll.hpp, inc/splitter.hpp).
// The library holds the fp32 instantiation; the templates exist so that reference call sites
// such as `SparseCoo<COMPUTETYPE>`, `CSR_Matrix<COMPUTETYPE>`, `preprocess<COMPUTETYPE>`
// (gpu_kernels.cu:1290-1292,1464) keep compiling with COMPUTETYPE = float.
// ---------------------------------------------------------------------------------------
#include <type_traits>
#include <vector>

template <class DType>
struct SparseCoo {
    static_assert(std::is_same<DType, float>::value, "libcutespmm implements the fp32 instantiation");
    int dimY = 0, dimX = 0, nnz = 0;
    int *rows = nullptr, *cols = nullptr;
    DType *values = nullptr;
    SparseCoo() = default;
    explicit SparseCoo(const std::string &FilePath)                        // inc/SparseCoo.hpp:91-157
    {
        cute::check(cute_coo_read(FilePath.c_str(), &raw_), "SparseCoo");
        sync();
    }
    SparseCoo(int dY, int dX, int /*nnz*/) { raw_.dimY = dY; raw_.dimX = dX; sync(); }   // :158-169
    explicit SparseCoo(const cute_coo &owned) : raw_(owned) { sync(); }
    void Insert_Next(int row, int col, DType val)                           // :243-248
    {
        if (!grown_) {   // move what a file or the library supplied into growable storage, once
            r_.assign(raw_.rows, raw_.rows + raw_.nnz);
            c_.assign(raw_.cols, raw_.cols + raw_.nnz);
            v_.assign(raw_.values, raw_.values + raw_.nnz);
            cute_coo_release(&raw_);
        }
        r_.push_back(row); c_.push_back(col); v_.push_back(val);
        raw_.dimY = dimY; raw_.dimX = dimX;
        raw_.nnz = int(r_.size());
        rows = raw_.rows = r_.data(); cols = raw_.cols = c_.data(); values = raw_.values = v_.data();
        nnz = raw_.nnz;
        grown_ = true;
    }
    void prepare_for_cusparse() {}                                          // :250-261: the arrays are already SoA
    void save_mtx(const std::string &path) const { cute::check(cute_coo_save_mtx(&raw_, path.c_str()), "save_mtx"); }
    int getX() const { return dimX; }
    int getY() const { return dimY; }
    const cute_coo &raw() const { return raw_; }
    ~SparseCoo() { if (!grown_) cute_coo_release(&raw_); }
    SparseCoo(const SparseCoo &) = delete;
    SparseCoo &operator=(const SparseCoo &) = delete;

private:
    cute_coo raw_{};
    std::vector<int> r_, c_;
    std::vector<DType> v_;
    bool grown_ = false;
    void sync() { dimY = raw_.dimY; dimX = raw_.dimX; nnz = raw_.nnz; rows = raw_.rows; cols = raw_.cols; values = raw_.values; }
};

template <class DType>
struct CSR_Matrix {
    static_assert(std::is_same<DType, float>::value, "libcutespmm implements the fp32 instantiation");
    int nrows = 0, ncols = 0, nnz = 0;
    DType *values = nullptr;
    int *cols = nullptr, *rowPtr = nullptr;
    int R = 0, C = 0, BCSR_nrows = 0, BCSR_ncols = 0, BCSR_nblks = 0;       // valid after to_BCSR (inc/CSR.hpp:52-60)
    DType *BCSR_values = nullptr;
    int *BCSR_cols = nullptr, *BCSR_rowPtr = nullptr;
    explicit CSR_Matrix(SparseCoo<DType> &S) { coo2CSR(S); }               // inc/CSR.hpp:68-71
    void coo2CSR(SparseCoo<DType> &S)                                       // :162-187
    {
        cute_csr_i32_release(&raw_);
        cute::check(cute_coo_to_csr(&S.raw(), &raw_), "coo2CSR");
        nrows = raw_.nrows; ncols = raw_.ncols; nnz = raw_.nnz; values = raw_.values; cols = raw_.cols; rowPtr = raw_.rowPtr;
    }
    template <class T> void ToDense(T *dense) const                         // :315-329
    {
        for (int r = 0; r < nrows; ++r)
            for (int e = rowPtr[r]; e < rowPtr[r + 1]; ++e) dense[size_t(r) * size_t(ncols) + size_t(cols[e])] = T(values[e]);
    }
    int csr_count_blocks(int R_, int C_) const                              // :728-743
    {
        int64_t n = cute_csr_count_blocks(&raw_, R_, C_);
        if (n < 0) throw cute::Error(int(n), "csr_count_blocks");
        return int(n);
    }
    void to_BCSR(int R_, int C_)                                            // :760-810
    {
        cute_bcsr_release(&bcsr_);
        cute::check(cute_csr_to_bcsr(&raw_, R_, C_, &bcsr_), "to_BCSR");
        R = bcsr_.R; C = bcsr_.C; BCSR_nrows = bcsr_.nrows; BCSR_ncols = bcsr_.ncols; BCSR_nblks = bcsr_.nblks;
        BCSR_values = bcsr_.values; BCSR_cols = bcsr_.cols; BCSR_rowPtr = bcsr_.rowPtr;
    }
    const cute_csr_i32 &raw() const { return raw_; }
    ~CSR_Matrix() { cute_csr_i32_release(&raw_); cute_bcsr_release(&bcsr_); }
    CSR_Matrix(const CSR_Matrix &) = delete;
    CSR_Matrix &operator=(const CSR_Matrix &) = delete;

private:
    cute_csr_i32 raw_{};
    cute_bcsr bcsr_{};
};

template <class DType>
class preprocess {                                                          // inc/prepareBlkEll.hpp:15-291
    static_assert(std::is_same<DType, float>::value, "libcutespmm implements the fp32 instantiation");

public:
    preprocess(CSR_Matrix<DType> *A_CSR, int BlockSize) : ncols_(A_CSR->ncols)
    {
        cute::check(cute_blocked_ell_build(&A_CSR->raw(), BlockSize, &e_), "preprocess");
    }
    ~preprocess() { cute_blocked_ell_dev_free(dev_); cute_blocked_ell_release(&e_); }
    void blockedELLToDense(DType *dense) { cute::check(cute_blocked_ell_to_dense(&e_, ncols_, dense), "blockedELLToDense"); }
    // C[height*BlockSize x N] (+)= ELL . B[ncols x N] on the GPU, device pointers; the place of the
    // cusparseSpMM call on a Blocked-ELL descriptor in the reference's harness (gpu_kernels.cu:166-223).
    void spmm(const DType *dB, DType *dC, unsigned int N, bool accumulate = false, void *stream = nullptr)
    {
        if (!dev_) cute::check(cute_blocked_ell_upload(&e_, &dev_), "Blocked-ELL upload");
        cute::check(cute_blocked_ell_spmm(dev_, dB, dC, N, accumulate ? 1 : 0, stream), "Blocked-ELL SpMM");
    }
    int *get_ellColIdx() { return e_.ellColIdx; }
    int get_ellColIdx_height() { return e_.height; }
    int get_ellColIdx_width() { return e_.width; }
    DType *get_ellValues() { return e_.ellValues; }
    int get_num_blocks() { return e_.numBlocks; }
    int get_num_elems() { return e_.numElems; }
    preprocess(const preprocess &) = delete;
    preprocess &operator=(const preprocess &) = delete;

private:
    cute_blocked_ell e_{};
    cute_blocked_ell_dev *dev_ = nullptr;
    int ncols_;
};

class Splitter {                                                            // inc/splitter.hpp:14-187
public:
    Splitter(CSR_Matrix<float> *A_CSR, int tile_size, int NNZThreshold)
    {
        cute::check(cute_splitter_split(&A_CSR->raw(), tile_size, NNZThreshold, &s_), "Splitter");
        heavy_ = new SparseCoo<float>(s_.heavy);
        light_ = new SparseCoo<float>(s_.light);
        s_.heavy = cute_coo{};   // ownership moved into the two SparseCoo objects
        s_.light = cute_coo{};
    }
    ~Splitter() { delete heavy_; delete light_; }
    int get_total_tiles() { return s_.totalTiles; }
    int get_num_heavy_tiles() { return s_.numHeavyTiles; }
    int get_num_heavy_elems() { return s_.numHeavyElems; }
    int get_num_light_tiles() { return s_.numLightTiles; }
    int get_num_light_elems() { return s_.numLightElems; }
    SparseCoo<float> *get_heavyMatrix() { return heavy_; }
    SparseCoo<float> *get_lightMatrix() { return light_; }
    Splitter(const Splitter &) = delete;
    Splitter &operator=(const Splitter &) = delete;

private:
    cute_split s_{};
    SparseCoo<float> *heavy_ = nullptr, *light_ = nullptr;
};

// The hybrid of inc/SPMM.cuh:2528-2933 (GPU_Compute_Multi_Kernel*: dense part on the matrix cores, remainder on a
// plain kernel) as one object: heavy tiles by the Splitter's rule (NNZThreshold 0: the library's measured default)
// or by the block classifier's (inc/preprocess.hpp:172-193), multiplied into one C.
class HybridSpMM {
public:
    cute_hybrid_info info{};
    HybridSpMM(CSR_Matrix<float> *A_CSR, int tile_size = 16, int NNZThreshold = 0)
    {
        cute::check(cute_hybrid_create(&A_CSR->raw(), tile_size, NNZThreshold, CUTE_HYBRID_SPLITTER, 0.0f, 0.0f, &h_), "HybridSpMM");
        cute_hybrid_get_info(h_, &info);
    }
    HybridSpMM(CSR_Matrix<float> *A_CSR, int BlockSize, float deviation_threshold, float underloadDominance)
    {
        cute::check(cute_hybrid_create(&A_CSR->raw(), BlockSize, 0, CUTE_HYBRID_CLASSIFIER, deviation_threshold, underloadDominance, &h_),
                    "HybridSpMM");
        cute_hybrid_get_info(h_, &info);
    }
    // dB [ncols x N], dC [nrows x N]: device pointers; asynchronous on `stream`
    void run(const float *dB, float *dC, uint32_t N, void *stream = nullptr) { cute::check(cute_hybrid_spmm(h_, dB, dC, N, stream), "HybridSpMM::run"); }
    ~HybridSpMM() { cute_hybrid_free(h_); }
    HybridSpMM(const HybridSpMM &) = delete;
    HybridSpMM &operator=(const HybridSpMM &) = delete;

private:
    cute_hybrid *h_ = nullptr;
};

// Block statistics the reference's harness chooses its split threshold from (gpu_kernels.cu:1049-1186).
inline void GET_STATS(CSR_Matrix<float> *A_CSR, uint32_t blocksize, std::vector<float> &stats)
{
    if (stats.size() < 4) stats.resize(4);
    cute::check(cute_block_stats(&A_CSR->raw(), int32_t(blocksize), stats.data()), "GET_STATS");
}
inline float GET_ANXS(CSR_Matrix<float> *A_CSR, uint32_t blocksize, bool axis)
{
    float v = 0.0f;
    cute::check(cute_anxs(&A_CSR->raw(), int32_t(blocksize), axis ? 1 : 0, &v), "GET_ANXS");
    return v;
}
