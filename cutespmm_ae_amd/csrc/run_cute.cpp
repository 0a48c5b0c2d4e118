// run_cute -- single-GPU driver, the counterpart of the reference's main (run.cu:8-72).
//
//   run_cute <file.mtx | gen:CFG>  [--n 32,128,512] [--iters 20] [--keep-values] [--no-check]
//
// Reads (or generates) A, builds the HRPB once (timed, run.cu:17-20), fills B with seeded
// U(0,1) values (run.cu:24-27 uses rand()), then for every N (run.cu:16: 32, 128, 512)
// plans, launches, times with HIP events (3 warm-ups, `iters` timed launches, median) and --
// the ERROR_CHECK branch of run.cu:57-64 -- compares with the plain CSR kernel.  One JSON
// line per N on stdout: GFLOP/s = 2 nnz N / t, algorithmic GB/s and its share of 8 TB/s.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/cutespmm.hpp"

namespace {

struct DeviceBuffer {
    float *p = nullptr;
    explicit DeviceBuffer(size_t count)
    {
        if (hipMalloc(reinterpret_cast<void **>(&p), count * sizeof(float)) != hipSuccess)
            throw cute::Error(CUTE_ERR_HIP, "hipMalloc");
    }
    ~DeviceBuffer() { (void)hipFree(p); }
};

double median(std::vector<float> v)
{
    std::sort(v.begin(), v.end());
    return v.empty() ? 0.0 : v[v.size() / 2];
}

const unsigned kStock[6][4] = {{0, 0, 0, 0}, {1, 4096, 16, 0}, {2, 256, 0, 0}, {3, 8000, 200, 0}, {4, 17, 10, 0},
                               {5, 1048576, 32, 2048}};

}  // namespace

int main(int argc, char **argv)
{
    if (argc < 2) {
        std::fprintf(stderr, "usage: %s <file.mtx | gen:CFG> [--n 32,128,512] [--iters 20] [--keep-values] [--no-check]\n", argv[0]);
        return 2;
    }
    std::vector<unsigned> widths = {32, 128, 512};
    int iters = 20;
    bool keep_values = false, check = true;
    for (int i = 2; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--n" && i + 1 < argc) {
            widths.clear();
            for (char *tok = std::strtok(argv[++i], ","); tok; tok = std::strtok(nullptr, ",")) widths.push_back(unsigned(std::atoi(tok)));
        } else if (a == "--iters" && i + 1 < argc) iters = std::max(1, std::atoi(argv[++i]));
        else if (a == "--keep-values") keep_values = true;
        else if (a == "--no-check") check = false;
        else { std::fprintf(stderr, "unknown argument %s\n", a.c_str()); return 2; }
    }
    try {
        std::string src = argv[1];
        MTX_READER *reader;
        if (src.rfind("gen:", 0) == 0) {
            int cfg = std::atoi(src.c_str() + 4);
            if (cfg < 1 || cfg > 5) throw cute::Error(CUTE_ERR_ARG, "gen:CFG needs 1..5");
            cute_csr csr;
            cute::check(cute_gen_matrix(int(kStock[cfg][0]), 0xC07E5B00ull + cfg, kStock[cfg][1], kStock[cfg][2], kStock[cfg][3], &csr), "cute_gen_matrix");
            reader = new MTX_READER(csr);
        } else {
            reader = new MTX_READER(src, keep_values);
            reader->sort_rows();   // HRPB needs sorted rows; the reference assumes its inputs are
        }
        const unsigned M = reader->M, K = reader->K, nnz = reader->nnz;
        auto t0 = std::chrono::steady_clock::now();
        HRPB hrpb(M, K, reader->rowPtr, reader->cols, reader->vals);
        const double prep_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();

        const unsigned maxN = *std::max_element(widths.begin(), widths.end());
        std::vector<float> b(size_t(K) * maxN), c_host, c_ref;
        for (unsigned N : widths) {
            cute::check(cute_gen_dense(0xB0B0ull + N, 0, uint64_t(K) * N, b.data()), "cute_gen_dense");
            DeviceBuffer dB(size_t(K) * N), dC(size_t(M) * N);
            if (hipMemcpy(dB.p, b.data(), size_t(K) * N * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
                throw cute::Error(CUTE_ERR_HIP, "hipMemcpy B");
            SPMM_TC spmm(M, K, N, hrpb);
            spmm.run(dB.p, dC.p);
            std::vector<float> ms(size_t(iters), 0.0f);
            cute::check(cute_spmm_time(spmm.plan(), dB.p, dC.p, nullptr, 3, iters, ms.data()), "cute_spmm_time");
            const double t_ms = median(ms);
            double ref_metric = -1.0, back_err = -1.0, csr_ms = -1.0;
            if (check) {
                c_host.resize(size_t(M) * N);
                c_ref.assign(size_t(M) * N, 0.0f);
                if (hipMemcpy(c_host.data(), dC.p, c_host.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
                    throw cute::Error(CUTE_ERR_HIP, "hipMemcpy C");
                csr_ms = GPU_CSR_cuSPARSE_NEW(reader->rowPtr, reader->cols, reader->vals, nnz, b.data(), c_ref.data(), M, K, N, 5);
                ref_metric = check_gemm_correctness_coo(c_ref.data(), c_host.data(), M, N);
                back_err = cute_backward_error(reader->rowPtr, reader->cols, reader->vals, b.data(), c_ref.data(), c_host.data(), M, N);
            }
            const double flops = 2.0 * double(nnz) * N;
            const double bytes = double(nnz) * 8 + (double(M) + 1) * 4 + double(K) * N * 4 + double(M) * N * 4;
            std::printf("{\"matrix\": \"%s\", \"M\": %u, \"K\": %u, \"nnz\": %u, \"N\": %u, \"blocks\": %u, \"bricks\": %u, "
                        "\"brick_density\": %.4f, \"prep_ms\": %.3f, \"chunks\": %u, \"atomic_chunks\": %u, \"sparse_panels\": %u, "
                        "\"kernel_us\": %.2f, \"gflops\": %.1f, \"algorithmic_GBps\": %.1f, \"hbm_roofline_frac\": %.4f, "
                        "\"csr_kernel_us\": %.2f, \"max_rel_err\": %.3e, \"backward_err\": %.3e}\n",
                        src.c_str(), M, K, nnz, N, hrpb.host().numBlocks, hrpb.num_bricks, hrpb.block_density, prep_ms,
                        spmm.info.numChunks, spmm.info.numAtomicChunks, spmm.info.numRowPanelsSparse, t_ms * 1e3,
                        flops / (t_ms * 1e-3) / 1e9, bytes / (t_ms * 1e-3) / 1e9, bytes / (t_ms * 1e-3) / 8e12,
                        csr_ms * 1e3, ref_metric, back_err);
            std::fflush(stdout);
        }
        delete reader;
    } catch (const std::exception &e) {
        std::fprintf(stderr, "run_cute: %s\n", e.what());
        return 1;
    }
    return 0;
}
