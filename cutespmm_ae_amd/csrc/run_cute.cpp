// run_cute -- single-GPU driver, the counterpart of the reference's main (run.cu:8-72).
//
//   run_cute <file.mtx | gen:CFG>  [--n 32,128,512] [--iters 20] [--keep-values] [--no-check] [--cache FILE] [--extras]
//
// Reads (or generates) A, builds the HRPB once (timed, run.cu:17-20; with --cache the converted
// matrix is written to FILE, and read from it instead when FILE already exists), fills B with seeded
// U(0,1) values (run.cu:24-27 uses rand()), then for every N (run.cu:16: 32, 128, 512)
// plans, launches, times with HIP events (3 warm-ups, then `iters` launches inside one event pair, the median of three such pairs) and --
// the ERROR_CHECK branch of run.cu:57-64 -- compares with the plain CSR kernel.  One JSON
// line per N on stdout: GFLOP/s = 2 nnz N / t, algorithmic GB/s and its share of 8 TB/s.
// --extras also takes the two routes the reference's driver does not have, per N: the format built on the device from
// the CSR arrays that live there (HRPB_DEVICE; its product, run with the partial tiles in a caller's buffer, must equal
// the first one bit for bit) and the hybrid of inc/SPMM.cuh:2528-2933 (HybridSpMM: heavy tiles on the matrix cores,
// the remainder on the row kernel; checked with the reference's metric).
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

const unsigned kStock[6][4] = {{0, 0, 0, 0}, {1, 4096, 16, 0}, {2, 256, 0, 0}, {3, 8000, 200, 0}, {4, 17, 10, 0},
                               {5, 1048576, 32, 2048}};

}  // namespace

int main(int argc, char **argv)
{
    if (argc < 2) {
        std::fprintf(stderr, "usage: %s <file.mtx | gen:CFG> [--n 32,128,512] [--iters 20] [--keep-values] [--no-check] [--cache FILE]\n", argv[0]);
        return 2;
    }
    std::vector<unsigned> widths = {32, 128, 512};
    int iters = 20;
    double ramp_ms = 30.0;     // launches before anything is timed: the GPU needs some milliseconds of work to reach its steady clocks
    bool keep_values = false, check = true, extras = false;
    std::string cache_file;
    for (int i = 2; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--n" && i + 1 < argc) {
            widths.clear();
            for (char *tok = std::strtok(argv[++i], ","); tok; tok = std::strtok(nullptr, ",")) widths.push_back(unsigned(std::atoi(tok)));
        } else if (a == "--iters" && i + 1 < argc) iters = std::max(1, std::atoi(argv[++i]));
        else if (a == "--ramp-ms" && i + 1 < argc) ramp_ms = std::max(0.0, std::atof(argv[++i]));
        else if (a == "--keep-values") keep_values = true;
        else if (a == "--no-check") check = false;
        else if (a == "--extras") extras = true;
        else if (a == "--cache" && i + 1 < argc) cache_file = argv[++i];
        else { std::fprintf(stderr, "unknown argument %s\n", a.c_str()); return 2; }
    }
    try {
        std::string src = argv[1];
        MTX_READER *reader = nullptr;
        HRPB *format = nullptr;
        bool from_cache = false;
        {   // bring the HIP runtime up before anything is timed: the first device call costs tens of milliseconds
            int cus = 0, wave = 0;
            char arch[64];
            cute::check(cute_device_info(&cus, &wave, arch, sizeof arch), "cute_device_info");
            std::vector<float> host(1u << 18, 0.0f);   // the first allocation and the first copy pay for the runtime's set-up
            void *warm = nullptr;
            if (hipMalloc(&warm, host.size() * sizeof(float)) != hipSuccess ||
                hipMemcpy(warm, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess ||
                hipDeviceSynchronize() != hipSuccess)
                throw cute::Error(CUTE_ERR_HIP, "device warm-up");
            (void)hipFree(warm);
        }
        auto t0 = std::chrono::steady_clock::now();
        if (!cache_file.empty()) {
            if (FILE *probe = std::fopen(cache_file.c_str(), "rb")) {
                std::fclose(probe);
                format = new HRPB(cache_file.c_str());
                from_cache = true;
            }
        }
        if (!format) {
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
            t0 = std::chrono::steady_clock::now();     // as run.cu:17-20: the conversion alone
            format = new HRPB(reader->M, reader->K, reader->rowPtr, reader->cols, reader->vals);
        }
        const double prep_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        if (!cache_file.empty() && !from_cache) format->save(cache_file.c_str());
        HRPB &hrpb = *format;
        const unsigned M = hrpb.M, K = hrpb.K, nnz = hrpb.numNNZ;

        const unsigned maxN = *std::max_element(widths.begin(), widths.end());
        std::vector<float> b(size_t(K) * maxN), c_host, c_ref;
        for (unsigned N : widths) {
            cute::check(cute_gen_dense(0xB0B0ull + N, 0, uint64_t(K) * N, b.data()), "cute_gen_dense");
            DeviceBuffer dB(size_t(K) * N), dC(size_t(M) * N);
            if (hipMemcpy(dB.p, b.data(), size_t(K) * N * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
                throw cute::Error(CUTE_ERR_HIP, "hipMemcpy B");
            SPMM_TC spmm(M, K, N, hrpb.blockedRowPtr);                                              // run.cu:45
            spmm.run(hrpb.blocksDevice, dB.p, dC.p, hrpb.activeColsDevice, hrpb.sizePtrDevice);     // run.cu:46-50
            // timed like the comparison path (spmm.cu:941-953): warm-up launches, then `iters` launches
            // between one pair of events, divided by `iters` -- after `ramp_ms` of the same launches, for
            // both columns of the table alike
            auto time_launches = [&](auto &&launch) {
                const auto ramp_end = std::chrono::steady_clock::now() + std::chrono::duration<double, std::milli>(ramp_ms);
                while (std::chrono::steady_clock::now() < ramp_end) {
                    for (int w = 0; w < 20; ++w) launch();
                    if (hipDeviceSynchronize() != hipSuccess) throw cute::Error(CUTE_ERR_HIP, "ramp");
                }
                for (int w = 0; w < 3; ++w) launch();
                hipEvent_t e0, e1;
                if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) throw cute::Error(CUTE_ERR_HIP, "hipEventCreate");
                // three such brackets, the median reported: launches of a few microseconds scatter by 10-20 % from
                // one bracket to the next
                double bracket_ms[3];
                for (double &ms : bracket_ms) {
                    (void)hipEventRecord(e0, nullptr);
                    for (int it = 0; it < iters; ++it) launch();
                    (void)hipEventRecord(e1, nullptr);
                    float total_ms = 0.0f;
                    if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&total_ms, e0, e1) != hipSuccess)
                        throw cute::Error(CUTE_ERR_HIP, "timing");
                    ms = double(total_ms) / iters;
                }
                (void)hipEventDestroy(e0);
                (void)hipEventDestroy(e1);
                std::sort(bracket_ms, bracket_ms + 3);
                return bracket_ms[1];
            };
            const double t_ms = time_launches([&] { spmm.run(dB.p, dC.p); });
            double ref_metric = -1.0, back_err = -1.0, csr_ms = -1.0;
            if (check) {
                c_host.resize(size_t(M) * N);
                c_ref.assign(size_t(M) * N, 0.0f);
                if (hipMemcpy(c_host.data(), dC.p, c_host.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
                    throw cute::Error(CUTE_ERR_HIP, "hipMemcpy C");
                (void)GPU_CSR_cuSPARSE_NEW(hrpb.rowPtr, hrpb.cols, hrpb.vals, nnz, b.data(), c_ref.data(), M, K, N, 1);
                // the CSR kernel's time: same kernel on the uploaded CSR copy, same timing protocol as above
                const uint32_t *dRowPtr = nullptr, *dCols = nullptr;
                const float *dVals = nullptr;
                cute::check(cute_hrpb_dev_csr(hrpb.device, &dRowPtr, &dCols, &dVals), "cute_hrpb_dev_csr");
                DeviceBuffer dC2(size_t(M) * N);
                csr_ms = time_launches([&] {
                    cute::check(cute_csr_spmm_dev(2, dRowPtr, dCols, dVals, dB.p, dC2.p, M, N, nullptr), "cute_csr_spmm_dev");
                });
                ref_metric = check_gemm_correctness_coo(c_ref.data(), c_host.data(), M, N);
                back_err = cute_backward_error(hrpb.rowPtr, hrpb.cols, hrpb.vals, b.data(), c_ref.data(), c_host.data(), M, N);
            }
            int device_built_equal = -1;
            double hybrid_metric = -1.0;
            unsigned hybrid_heavy = 0;
            if (extras && check) {
                const uint32_t *dRowPtr = nullptr, *dCols = nullptr;
                const float *dVals = nullptr;
                cute::check(cute_hrpb_dev_csr(hrpb.device, &dRowPtr, &dCols, &dVals), "cute_hrpb_dev_csr");
                HRPB_DEVICE on_device(M, K, nnz, dRowPtr, dCols, dVals);
                SPMM_TC spmm2(M, K, N, on_device);
                DeviceBuffer dC3(size_t(M) * N), scratch(size_t(spmm2.scratch_bytes() / sizeof(float)) + 64);
                spmm2.run(dB.p, dC3.p, nullptr, scratch.p, spmm2.scratch_bytes());
                std::vector<float> c3(size_t(M) * N);
                if (hipMemcpy(c3.data(), dC3.p, c3.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
                    throw cute::Error(CUTE_ERR_HIP, "hipMemcpy C (device-built)");
                device_built_equal = std::memcmp(c3.data(), c_host.data(), c3.size() * sizeof(float)) == 0 ? 1 : 0;
                SparseCoo<float> coo(static_cast<int>(M), static_cast<int>(K), static_cast<int>(nnz));
                for (unsigned r = 0; r < M; ++r)
                    for (unsigned e = hrpb.rowPtr[r]; e < hrpb.rowPtr[r + 1]; ++e) coo.Insert_Next(int(r), int(hrpb.cols[e]), hrpb.vals[e]);
                CSR_Matrix<float> csr(coo);
                HybridSpMM hybrid(&csr);
                hybrid.run(dB.p, dC3.p, N);
                if (hipMemcpy(c3.data(), dC3.p, c3.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
                    throw cute::Error(CUTE_ERR_HIP, "hipMemcpy C (hybrid)");
                hybrid_metric = check_gemm_correctness_coo(c_ref.data(), c3.data(), M, N);
                hybrid_heavy = hybrid.info.heavyTiles;
            }
            const double flops = 2.0 * double(nnz) * N;
            const double bytes = double(nnz) * 8 + (double(M) + 1) * 4 + double(K) * N * 4 + double(M) * N * 4;
            std::printf("{\"matrix\": \"%s\", \"M\": %u, \"K\": %u, \"nnz\": %u, \"N\": %u, \"blocks\": %u, \"bricks\": %u, "
                        "\"brick_density\": %.4f, \"prep_ms\": %.3f, \"from_cache\": %s, \"chunks\": %u, \"atomic_chunks\": %u, \"sparse_panels\": %u, "
                        "\"kernel_us\": %.2f, \"gflops\": %.1f, \"algorithmic_GBps\": %.1f, \"hbm_roofline_frac\": %.4f, "
                        "\"csr_kernel_us\": %.2f, \"max_rel_err\": %.3e, \"backward_err\": %.3e, "
                        "\"device_built_equal\": %d, \"hybrid_max_rel_err\": %.3e, \"hybrid_heavy_tiles\": %u}\n",
                        src.c_str(), M, K, nnz, N, hrpb.host().numBlocks, hrpb.num_bricks, hrpb.block_density, prep_ms, from_cache ? "true" : "false",
                        spmm.info.numChunks, spmm.info.numAtomicChunks, spmm.info.numRowPanelsSparse, t_ms * 1e3,
                        flops / (t_ms * 1e-3) / 1e9, bytes / (t_ms * 1e-3) / 1e9, bytes / (t_ms * 1e-3) / 8e12,
                        csr_ms * 1e3, ref_metric, back_err, device_built_equal, hybrid_metric, hybrid_heavy);
            std::fflush(stdout);
        }
        delete format;
        delete reader;
    } catch (const std::exception &e) {
        std::fprintf(stderr, "run_cute: %s\n", e.what());
        return 1;
    }
    return 0;
}
