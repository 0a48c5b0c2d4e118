// membw_probe: what the memory system of one MI355X gives to the access patterns an SpMM launch is made of.
//
// Every figure is taken twice: "rotating" cycles through 20 buffer sets (1.6 GB, far more than the 256 MB
// Infinity Cache holds, so the operands come from HBM) and "one set" repeats on the same buffers (the
// Infinity Cache, and for 32 MB the L2s, serve the reads).  400 back-to-back launches between one pair of
// HIP events, best of three, after 600 warm-up launches.
//
// Patterns (4 096 wavefronts = the number of row panels of the 65 536-row benchmark matrix):
//   read only            each wavefront sums a private contiguous region (4 KB batches, four 16-byte loads per lane in flight)
//   write only           each wavefront fills 8 KB (one C tile of 16 rows x 128 floats)
//   read R then write 8  what an SpMM wavefront does to memory: all its reads, then its C tile
//   the same with fewer, longer wavefronts or as two launches of half the wavefronts
//   hipMemcpyAsync       the runtime's device-to-device copy
//
// Usage: membw_probe            (no arguments; prints one line per pattern and protocol)
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                                        \
    do {                                                                                \
        hipError_t e_ = (x);                                                            \
        if (e_ != hipSuccess) {                                                         \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(1);                                                               \
        }                                                                               \
    } while (0)

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr size_t kMiB = size_t(1) << 20;
constexpr size_t kSrcPerSet = 48 * kMiB, kDstPerSet = 32 * kMiB;
constexpr int kSets = 20;

// ITEMS times { read batches x 4 KB, write 8 KB } per wavefront; `never` is a value the sums cannot take, so the
// compiler has to keep the loads.
template <int ITEMS>
__global__ __launch_bounds__(256) void read_then_write(const f32x4 *__restrict__ src, f32x4 *__restrict__ dst, int batches, float never)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wave = blockIdx.x * 4u + (threadIdx.x >> 6);
#pragma unroll 1
    for (int p = 0; p < ITEMS; ++p) {
        const unsigned item = wave * ITEMS + p;
        const f32x4 *s = src + size_t(item) * batches * 256u + lane;
        f32x4 a0 = f32x4(0.f), a1 = f32x4(0.f), a2 = f32x4(0.f), a3 = f32x4(0.f);
        for (int b = 0; b < batches; ++b) {
            a0 += s[b * 256 + 0];
            a1 += s[b * 256 + 64];
            a2 += s[b * 256 + 128];
            a3 += s[b * 256 + 192];
        }
        f32x4 *d = dst + size_t(item) * 512u + lane;
        if (a0.x == never) a1.x = 1.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            f32x4 v = (r & 1) ? a1 : a0;
            v += (r & 2) ? a2 : a3;
            __builtin_nontemporal_store(v, d + r * 64);
        }
    }
}

__global__ __launch_bounds__(256) void read_only(const f32x4 *__restrict__ src, f32x4 *__restrict__ dst, int batches, float never)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wave = blockIdx.x * 4u + (threadIdx.x >> 6);
    const f32x4 *s = src + size_t(wave) * batches * 256u + lane;
    f32x4 a0 = f32x4(0.f), a1 = f32x4(0.f), a2 = f32x4(0.f), a3 = f32x4(0.f);
    for (int b = 0; b < batches; ++b) {
        a0 += s[b * 256 + 0];
        a1 += s[b * 256 + 64];
        a2 += s[b * 256 + 128];
        a3 += s[b * 256 + 192];
    }
    a0 += a1 + a2 + a3;
    if (a0.x == never) dst[wave] = a0;
}

__global__ __launch_bounds__(256) void write_only(f32x4 *__restrict__ dst, float x)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wave = blockIdx.x * 4u + (threadIdx.x >> 6);
    f32x4 *d = dst + size_t(wave) * 512u + lane;
#pragma unroll
    for (int r = 0; r < 8; ++r) __builtin_nontemporal_store(f32x4(x), d + r * 64);
}

}  // namespace

int main()
{
    char *src, *dst;
    CHECK(hipMalloc(&src, kSrcPerSet * kSets));
    CHECK(hipMalloc(&dst, kDstPerSet * kSets));
    CHECK(hipMemset(src, 0, kSrcPerSet * kSets));
    CHECK(hipMemset(dst, 0, kDstPerSet * kSets));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    auto S = [&](int set) { return reinterpret_cast<const f32x4 *>(src + kSrcPerSet * set); };
    auto D = [&](int set) { return reinterpret_cast<f32x4 *>(dst + kDstPerSet * set); };
    auto timeit = [&](const char *name, double bytes, auto launch) {
        for (int rotating = 1; rotating >= 0; --rotating) {
            int i = 0;
            for (int w = 0; w < 600; ++w) launch(rotating ? (i++ % kSets) : 0);
            CHECK(hipDeviceSynchronize());
            float best = 1e9f;
            for (int rep = 0; rep < 3; ++rep) {
                CHECK(hipEventRecord(e0, nullptr));
                for (int k = 0; k < 400; ++k) launch(rotating ? (i++ % kSets) : 0);
                CHECK(hipEventRecord(e1, nullptr));
                CHECK(hipEventSynchronize(e1));
                float ms;
                CHECK(hipEventElapsedTime(&ms, e0, e1));
                best = std::min(best, ms / 400.f * 1000.f);
            }
            std::printf("%-52s %s %7.2f us  %5.2f TB/s\n", name, rotating ? "rotating" : "one set ", best, bytes / best / 1e6);
        }
        std::fflush(stdout);
    };
    const double MB = double(kMiB);
    const float never = 3.f;      // the source is all zeros
    timeit("read only, 4096 wavefronts x 8 KB (33.6 MB)", 32 * MB,
           [&](int s) { hipLaunchKernelGGL(read_only, dim3(1024), dim3(256), 0, nullptr, S(s), D(s), 2, never); });
    timeit("read only, 4096 wavefronts x 12 KB (50.3 MB)", 48 * MB,
           [&](int s) { hipLaunchKernelGGL(read_only, dim3(1024), dim3(256), 0, nullptr, S(s), D(s), 3, never); });
    timeit("read only, 12288 wavefronts x 4 KB (50.3 MB)", 48 * MB,
           [&](int s) { hipLaunchKernelGGL(read_only, dim3(3072), dim3(256), 0, nullptr, S(s), D(s), 1, never); });
    timeit("write only, 4096 wavefronts x 8 KB (33.6 MB)", 32 * MB,
           [&](int s) { hipLaunchKernelGGL(write_only, dim3(1024), dim3(256), 0, nullptr, D(s), 1.f); });
    timeit("read 8 KB then write 8 KB, 4096 wavefronts (67.1 MB)", 64 * MB,
           [&](int s) { hipLaunchKernelGGL(read_then_write<1>, dim3(1024), dim3(256), 0, nullptr, S(s), D(s), 2, never); });
    timeit("read 12 KB then write 8 KB, 4096 wavefronts (83.9 MB)", 80 * MB,
           [&](int s) { hipLaunchKernelGGL(read_then_write<1>, dim3(1024), dim3(256), 0, nullptr, S(s), D(s), 3, never); });
    timeit("2 x (read 12 KB, write 8 KB), 2048 wavefronts", 80 * MB,
           [&](int s) { hipLaunchKernelGGL(read_then_write<2>, dim3(512), dim3(256), 0, nullptr, S(s), D(s), 3, never); });
    timeit("4 x (read 12 KB, write 8 KB), 1024 wavefronts", 80 * MB,
           [&](int s) { hipLaunchKernelGGL(read_then_write<4>, dim3(256), dim3(256), 0, nullptr, S(s), D(s), 3, never); });
    timeit("read 12 KB then write 8 KB, two launches of 2048", 80 * MB, [&](int s) {
        hipLaunchKernelGGL(read_then_write<1>, dim3(512), dim3(256), 0, nullptr, S(s), D(s), 3, never);
        hipLaunchKernelGGL(read_then_write<1>, dim3(512), dim3(256), 0, nullptr, S(s) + 2048 * 768, D(s) + 2048 * 512, 3, never);
    });
    timeit("hipMemcpyAsync device to device, 33.6 MB (67.1 MB moved)", 64 * MB,
           [&](int s) { (void)hipMemcpyAsync(D(s), S(s), 32 * kMiB, hipMemcpyDeviceToDevice, nullptr); });
    CHECK(hipDeviceSynchronize());
    CHECK(hipFree(src));
    CHECK(hipFree(dst));
    return 0;
}
