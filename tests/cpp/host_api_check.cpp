// Host-only use of the C++ mirror classes (include/cutespmm.hpp); prints one line that the
// Python test compares with the oracle and the recorded values.  No GPU call is made.
#include <cstdio>
#include <vector>

#include "cutespmm.hpp"

int main(int argc, char **argv)
{
    if (argc < 2) return 2;
    try {
        MTX_READER reader(argv[1]);
        HRPB hrpb(reader.M, reader.K, reader.rowPtr, reader.cols, reader.vals, /*upload=*/false);
        SparseCoo<float> coo(argv[1]);
        CSR_Matrix<float> csr(coo);
        preprocess<float> ell(&csr, 16);
        Splitter split(&csr, 16, 8);
        csr.to_BCSR(16, 4);
        std::vector<float> dense(size_t(ell.get_ellColIdx_height()) * 16 * size_t(csr.ncols), 0.0f), dense2(dense.size(), 0.0f);
        ell.blockedELLToDense(dense.data());
        csr.ToDense(dense2.data());
        size_t diff = 0;
        for (size_t i = 0; i < dense.size(); ++i) diff += dense[i] != dense2[i];
        SparseCoo<float> grown(4, 4, 0);
        grown.Insert_Next(1, 2, 3.0f);
        grown.Insert_Next(0, 1, 2.0f);
        CSR_Matrix<float> small(grown);
        std::printf("M=%u K=%u nnz=%u panels=%u blocks=%u words=%llu bricks=%u bcsr=%d ell=%dx%d ellblocks=%d tiles=%d heavy=%d/%d light=%d/%d "
                    "densediff=%zu grown=%d,%d\n",
                    reader.M, reader.K, reader.nnz, hrpb.numRowPanels, hrpb.blockedRowPtr[hrpb.numRowPanels], hrpb.dataStructSize,
                    hrpb.num_bricks, csr.BCSR_nblks, ell.get_ellColIdx_height(), ell.get_ellColIdx_width(), ell.get_num_blocks(),
                    split.get_total_tiles(), split.get_num_heavy_tiles(), split.get_num_heavy_elems(), split.get_num_light_tiles(),
                    split.get_num_light_elems(), diff, small.nnz, small.cols[0]);
        std::vector<float> stats(4);
        GET_STATS(&csr, 16, stats);
        std::printf("stats=%.9g,%.9g,%.9g,%.9g anxs=%.9g,%.9g\n", stats[0], stats[1], stats[2], stats[3], GET_ANXS(&csr, 16, true),
                    GET_ANXS(&csr, 16, false));
        if (argc > 2) {      // cache file: write, read back, compare every word
            hrpb.save(argv[2]);
            HRPB back(argv[2], /*upload=*/false);
            size_t bad = back.M != hrpb.M || back.K != hrpb.K || back.numNNZ != hrpb.numNNZ || back.dataStructSize != hrpb.dataStructSize;
            for (unsigned long long i = 0; i < hrpb.dataStructSize && !bad; ++i) bad += back.blocksData[i] != hrpb.blocksData[i];
            for (unsigned int i = 0; i < hrpb.numNNZ && !bad; ++i) bad += back.cols[i] != hrpb.cols[i] || back.vals[i] != hrpb.vals[i];
            std::printf("cache=%zu\n", bad);
        }
        {   // the registry behind the reference-shaped SPMM_TC constructor, and spmm_coo (inc.h:71-83)
            const bool found = HRPB::find(hrpb.blockedRowPtr) == &hrpb && HRPB::find(reader.rowPtr) == nullptr;
            bool gone;
            unsigned int *stale;
            {
                HRPB second(reader.M, reader.K, reader.rowPtr, reader.cols, reader.vals, /*upload=*/false);
                stale = second.blockedRowPtr;
                gone = HRPB::find(stale) == &second;
            }
            gone = gone && HRPB::find(stale) == nullptr;
            bool refused = false;
            try {
                SPMM_TC plan(reader.M, reader.K, 32, reader.rowPtr);      // not a format's blockedRowPtr
            } catch (const cute::Error &e) {
                refused = e.status == CUTE_ERR_ARG;
            }
            unsigned int rows[3] = {1, 0, 1}, cols[3] = {0, 1, 0};
            float vals[3] = {2.0f, 3.0f, 4.0f}, B[4] = {1.0f, 10.0f, 100.0f, 1000.0f}, C[4];
            spmm_coo(rows, cols, vals, B, C, 2, 2, 2, 3);
            const bool coo = C[0] == 300.0f && C[1] == 3000.0f && C[2] == 6.0f && C[3] == 60.0f;
            std::printf("registry=%d%d%d coo=%d fit=%d%d\n", int(found), int(gone), int(refused), int(coo),
                        cute_offsets_fit(4096, 4096, 16, 0, (1u << 20) * 16ull), cute_offsets_fit(4096, 4096, 16, 0, (1u << 20) * 16ull - 16));
        }
        try {
            MTX_READER missing("/nonexistent/file.mtx");
            return 3;
        } catch (const cute::Error &e) {
            if (e.status != CUTE_ERR_IO) return 4;
        }
    } catch (const std::exception &e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 1;
    }
    return 0;
}
