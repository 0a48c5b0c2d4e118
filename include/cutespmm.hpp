// cutespmm.hpp -- the reference's C++ host classes, re-stated over the C ABI of libcutespmm.
//
// Same class names, public fields and call sequence as the reference's driver uses
// (run.cu:11-62):   MTX_READER r(path);  HRPB hrpb(M, K, r.rowPtr, r.cols, r.vals);
//                   SPMM_TC spmm(M, K, N, hrpb);  spmm.run(dB, dC);
// Differences, all deliberate: every object frees what it owns; errors throw
// cute::Error instead of exit(-1) (inc.h:63-70) or a float-typed EXIT_FAILURE
// (spmm.cu:841-859); HRPB checks its preconditions; C need not be zeroed by the caller.
#pragma once
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
    cute_hrpb_dev *device = nullptr;  // stands for the four *Device pointers of data.cu:65-72

    HRPB(unsigned int M_, unsigned int K_, unsigned int *rowPtr_, unsigned int *cols_, float *vals_, bool upload = true)
        : cols(cols_), rowPtr(rowPtr_), vals(vals_), M(M_), K(K_), numRowPanels(M_ / CUTE_TM)
    {
        cute::check(cute_hrpb_build(M, K, rowPtr, cols, vals, &host_), "HRPB");
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
            if (rc != CUTE_OK) { cute_hrpb_host_release(&host_); throw cute::Error(rc, "HRPB upload"); }
        }
    }
    void freeDevice() { cute_hrpb_dev_free(device); device = nullptr; }   // data.cu:336-339
    const cute_hrpb_host &host() const { return host_; }
    ~HRPB() { freeDevice(); cute_hrpb_host_release(&host_); }
    HRPB(const HRPB &) = delete;
    HRPB &operator=(const HRPB &) = delete;

private:
    cute_hrpb_host host_{};
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
        if (!hrpb.device) throw cute::Error(CUTE_ERR_ARG, "SPMM_TC: HRPB has no device copy");
        cute::check(cute_spmm_plan_create(hrpb.device, N, tunables, &plan_), "SPMM_TC");
        cute_spmm_plan_info(plan_, &info);
        numRowPanelsSplit = info.numChunks;
    }
    // MatB [K x N], MatC [M x N]: device pointers; asynchronous on `stream`.
    void run(const float *MatB, float *MatC, void *stream = nullptr)
    {
        cute::check(cute_spmm_run(plan_, MatB, MatC, stream), "SPMM_TC::run");
    }
    cute_spmm_plan *plan() { return plan_; }
    ~SPMM_TC() { cute_spmm_plan_free(plan_); }
    SPMM_TC(const SPMM_TC &) = delete;
    SPMM_TC &operator=(const SPMM_TC &) = delete;

private:
    cute_spmm_plan *plan_ = nullptr;
};

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
