// Device side of libcutespmm: upload, plan, launch, plain CSR kernels, timing helpers.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <mutex>
#include <string>

#include "common.hpp"
#include "kernels.hip.hpp"
#include "build_kernels.hip.hpp"

using namespace cute;

namespace {

thread_local std::string g_hip_error;

// The planner's default thresholds (measured on the five benchmark matrices and on the reference's 43).
constexpr float kMinReuse = 1.25f;          // a panel with fewer nonzeros per B row the MFMA side would fetch goes to the row kernel
constexpr uint64_t kWideWindowBytes = 16ull << 20;   // ... whose window of B is wider than this (four L2s' worth)
constexpr float kWideReuse = 0.98f;          // ... the bar for products of 256 columns or more over large matrices (see cute_spmm_plan_create)
constexpr uint32_t kMaxRowForRows = 48;
constexpr uint32_t kMaxHubRows = 256;       // hub plans: B rows a work-group keeps in LDS (64 KiB of 256-byte pieces; two work-groups per CU)     // ... unless it holds a row longer than this: one lane group would serialise it
constexpr uint32_t kUnevenRowFloor = 16;     // row kernel vs MFMA kernel: a panel whose longest row exceeds this and ...
constexpr uint32_t kUnevenRowRatio = 2;      // ... this many mean rows of the panel goes to the MFMA kernel while rows share wavefronts
constexpr float kHybridFill = 0.15f;         // cute_hybrid: a tile goes to the Blocked-ELL part from this fill on (threshold 0)
constexpr uint64_t kSlotsPerBrick = 8;      // quad lists when the MFMA panels need fewer list slots per 16x4 brick, else brick tiles
// B and C together larger than the Infinity Cache: whatever the caller does between launches, their rows come
// from HBM.  There the brick kernel's wider row pieces (16 lanes x 16 bytes per row and column group, two groups
// per wavefront from N = 128 on) beat the quad kernel's 256-byte pieces by 20-25 % (9-point stencils of 0.25 to
// 1 million rows) -- as long as its matrix work, 32 cycles per brick and 16 columns however empty the brick,
// stays below the time the operands take to stream at 4 TB/s; on R-MAT graphs, where it is 1.4 to 1.7 times
// that, the two kernels are within 10 % of each other either way and the rule above keeps deciding.  While the
// operands fit the cache the quad kernel is level or ahead.
constexpr double kStreamBytesPerSecond = 4.0e12, kSimdCyclesPerSecond = 1024 * 2.4e9, kCyclesPerBrickTile = 32.0;

// Which MFMA kernel serves the panels that go to the matrix cores (1 brick tiles, 2 quad lists).
//   slots   list slots of the quad lists (pairs plus padding): the quad kernel pays 8 matrix cycles and one
//           256-byte piece of a B row per slot and 64 columns
//   bricks  16x4 bricks: the brick kernel pays 32 matrix cycles per brick and 16 columns, however empty the brick
//   blocks  16-column blocks: the brick kernel requests 16 row pieces per block (padding columns included)
// A launch fed from a cache is bound by what it issues, and the two kernels cross at about 8 slots per brick
// (measured on the benchmark matrices and on the reference's 43).  A launch fed from HBM is bound by the
// memory system, and what counts there is how many row pieces a kernel requests and how wide they are: the
// brick kernel asks for a B row once per panel, in pieces of 512 contiguous bytes from N = 128 on; the quad
// kernel once per 4-row group that uses it, in 256-byte pieces that two wavefronts request at different
// times.  Measured with operands no cache holds: 9-point stencils (1.25 slots per brick-kernel fetch) run
// 7-25 % faster through the brick kernel at 16 384 to 262 144 rows and N = 64..512, 5-point stencils (1.0)
// 5-8 % slower; from a cache the quad kernel is level or up to 20 % ahead on both.  So unless the caller
// says that the operands stay cache-resident (operand_residency = 2, a tight loop over the same buffers that
// fit the Infinity Cache), a matrix whose quad lists need more than 1.1 fetches per brick-kernel fetch goes to
// the brick kernel -- as long as its matrix work stays below the time the operands take to stream at 4 TB/s
// (on R-MAT graphs it is 1.4-1.7 times that, and the quad kernel keeps them).
int choose_mfma_shape(uint64_t slots, uint64_t bricks, uint64_t blocks, uint64_t rows_and_cols, uint64_t nnz, uint32_t N,
                      uint32_t residency, uint64_t cache_bytes)
{
    int shape = slots < kSlotsPerBrick * bricks ? 2 : 1;
    const bool resident = residency == 2 && rows_and_cols * N * sizeof(float) <= cache_bytes;
    if (shape == 2 && !resident && slots * 10u > blocks * 16u * 11u) {
        const double matrix_s = double(bricks) * double((N + 15u) / 16u) * kCyclesPerBrickTile / kSimdCyclesPerSecond;
        const double stream_s = (double(rows_and_cols) * N * 4.0 + double(nnz) * 8.0) / kStreamBytesPerSecond;
        if (matrix_s <= stream_s) shape = 1;
    }
    return shape;
}

inline int hip_fail(hipError_t e, const char *what, int line)
{
    g_hip_error = std::string(hipGetErrorString(e)) + " (" + what + ", device.hip:" + std::to_string(line) + ")";
    return CUTE_ERR_HIP;
}
#define HIP_TRY(expr)                                                    \
    do {                                                                 \
        hipError_t e_ = (expr);                                          \
        if (e_ != hipSuccess) return hip_fail(e_, #expr, __LINE__);      \
    } while (0)

struct DeviceContext {
    int status = CUTE_ERR_NO_DEVICE;
    int device = 0;
    int num_cus = 0;
    int wave_size = 0;
    // What the planner assumes about the part of the chip this device is.  A whole MI355X (SPX mode) shows 256
    // compute units in 8 XCDs of 32, each XCD with its own 4 MiB L2, and 256 MiB of Infinity Cache; in the
    // partitioned modes a device is 4, 2 or 1 of those XCDs with its share of the cache.  The kernels' mapping of
    // work-groups to contiguous panel ranges is written for 8 XCDs and stays a valid, locality-preserving order
    // on fewer (a device with x XCDs walks 8/x ranges per XCD); the model of where wavefronts land, which only
    // orders work items, is used on the whole chip alone.
    int num_xcds = 8;
    bool whole_chip = false;
    uint64_t cache_bytes = 256ull << 20;
    std::string arch;
};

// The library is written for gfx950 only; any other device is refused, loudly.
const DeviceContext &context()
{
    static DeviceContext ctx = [] {
        DeviceContext c;
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
            g_hip_error = "no HIP device visible";
            return c;
        }
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return c;
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return c;
        c.device = dev;
        c.num_cus = prop.multiProcessorCount;
        c.wave_size = prop.warpSize;
        c.arch = prop.gcnArchName;
        if (c.arch.rfind("gfx950", 0) != 0) {
            g_hip_error = "device is " + c.arch + ", this library is built for gfx950 only";
            return c;
        }
        if (c.num_cus > 0 && c.num_cus % 32 == 0 && c.num_cus / 32 <= 8) c.num_xcds = c.num_cus / 32;
        c.whole_chip = c.num_cus == 256;
        c.cache_bytes = (256ull << 20) * uint64_t(c.num_xcds) / 8u;
        c.status = CUTE_OK;
        return c;
    }();
    return ctx;
}

// Scratch for cute_spmm_run_static: the partial tiles of cut panels, for callers that cannot allocate.
// One copy per GPU, part of the loaded code object, held until the process ends.  In host code the name
// of the array is only a handle for hipGetSymbolAddress -- never a device address.
static __device__ __align__(256) unsigned char scratch[CUTE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void **out)
{
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return CUTE_ERR_ARG;
    std::lock_guard<std::mutex> g(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return CUTE_OK;
}

template <class T>
int upload(T **dst, const T *src, uint64_t count)
{
    *dst = nullptr;
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(dst), std::max<uint64_t>(count, 1) * sizeof(T)));
    if (count) HIP_TRY(hipMemcpy(*dst, src, count * sizeof(T), hipMemcpyHostToDevice));
    return CUTE_OK;
}

}  // namespace

struct cute_hrpb_dev {
    uint32_t M = 0, K = 0, nnz = 0, P = 0, nb = 0;
    uint64_t numVals = 0, bytes = 0;
    // Of the two MFMA layouts only the one the planner's default rules would pick for this matrix is built by
    // the upload (none if every panel would go to the row kernel); the other is built from the device copy of
    // the CSR arrays the first time a plan asks for it.  `lock` guards those late builds.
    std::mutex lock;
    bool haveBricks = false, haveQuads = false;
    uint32_t *dHdr = nullptr;           // brick tiles: one 128-byte header line per block
    float *dVals = nullptr;             // brick tiles: values in lane order, then 64 zeros
    uint32_t *dRowPtr = nullptr, *dCols = nullptr;
    float *dCsrVals = nullptr;
    uint32_t *dQRecs = nullptr;         // quad lists: one record per group (16 columns, slot mask, first value)
    float *dQVals = nullptr;            // quad lists: the occupied value slots in lane order, then 64 zeros
    uint64_t numQuadVals = 0;
    uint64_t numGroups = 0;
    std::vector<uint32_t> brp;          // host copy of blockedRowPtr
    std::vector<uint32_t> qgp;          // the quad lists' groupPtr (known from the census, before the lists are built)
    std::vector<uint32_t> stripPairs;   // length of the merged column list of every 4-row strip
    uint32_t quadRows = CUTE_TM;        // rows per list unit: 16 (lockstep lists per panel) or 4 (strips)
    uint64_t quadPairs = 0;             // occupied (row group, column) pairs
    std::vector<uint32_t> panelNnz;     // nonzeros per row panel
    std::vector<uint32_t> panelCols;    // active columns per row panel
    std::vector<uint32_t> panelMaxRow;  // longest row of each panel
    std::vector<uint32_t> panelSpan;    // width of each panel's column window (last column - first column + 1)
};

struct cute_spmm_plan {
    const cute_hrpb_dev *d = nullptr;
    cute_plan_info info{};
    int vec = 4, ng = 1;                // brick kernel shape
    int pipeline = 1;                   // 1: rolling variant, 2: pipelined variant
    int shape = 2;                      // MFMA kernel: 1 16x16x4 bricks, 2 4x4x1 quad lists
    bool bf16x3 = false;                // brick kernel on the bf16 matrix pipeline (three products of bf16 hi/lo parts)
    int rows_vec = 4, rows_logl = 6;    // row kernel shape
    uint32_t rows_slabs = 1;
    uint4 *dChunks = nullptr;
    uint32_t *dHeads = nullptr;         // quad kernels: per chunk, the descriptor and the record of its first group
    // hub plans: the most referenced B rows are staged in LDS by persistent work-groups (hrpb_quad_hub_f32)
    uint32_t numHub = 0;
    uint32_t *dHubRows = nullptr;       // the hub rows' column ids, slot order
    uint32_t *dHubRecs = nullptr;       // the plan's copy of the quad records, hub columns replaced by their slots
    // panels (or 4-row strips) cut into several chunks: each chunk stores a partial tile, reduce_partials adds them
    uint4 *dFixups = nullptr;           // {panel or strip, first piece, pieces, -}
    uint32_t numFixups = 0;
    uint32_t reduceBlocksY = 1;         // blocks of reduce_partials along a tile: enough for the tile with the most pieces
    uint32_t unitRows = CUTE_TM;        // rows of one panel / strip / piece
    float *dPartials = nullptr;         // pieces x unitRows rows of N floats; owned by the plan, so a plan runs on one stream at a time
    uint64_t partialBytes = 0;
    void *staticScratch = nullptr;      // device address of the library's static scratch array on the plan's device
    uint4 *dRowList = nullptr;          // rows of the sparse path with their row pointers: {row, first entry, end, 0}
    uint32_t numRows = 0;
    cute_dev::XcdRanges rowRanges{};   // row-kernel blocks of each XCD, balanced by nonzeros
    uint32_t rowBlocksPerXcd = 0;       // longest of those ranges
};

namespace {

// Deals the MFMA work items to the SIMDs by length.  When a launch fits on the device at once, nothing balances
// it afterwards: every wavefront is placed when the launch starts, and a SIMD that was handed three long panels
// keeps the whole launch waiting.  Where the work-groups land is regular (observed with the hardware id
// registers; nothing but speed depends on it): work-group g goes to XCD g % 8; the s-th work-group an XCD
// receives (x fastest, then the slabs) runs on its CU s % (CUs per XCD); and wavefront w of that work-group
// shares a SIMD with wavefront (w + 1) % 4 of the work-group the same CU received one round earlier.  So
// position (k, w) of an XCD's part of the list, in slab y, counts on SIMD lane (w + s / CUs) % 4 of CU s % CUs
// with s = y * groups_per_xcd + k.  Longest first, every item takes the free position that keeps the fullest
// SIMD it touches lowest (ties: the earliest position, so equal items stay in panel order and keep sharing B
// rows in the L1).  The new order is used only if the model says it shortens the fullest SIMD by 3 % or more.
// An item costs its length plus a fixed two units (descriptor, first operands, the store).
bool deal_chunks(std::vector<uint4> &chunks, uint32_t num_slabs, uint32_t cus_per_xcd, uint32_t waves_per_simd, bool force)
{
    const uint32_t wpg = cute_dev::kWavesPerGroup;
    if (cus_per_xcd == 0 || wpg != 4) return false;
    const uint64_t resident = uint64_t(cus_per_xcd) * cute_dev::kNumXcd * 4u * waves_per_simd;
    if (uint64_t(chunks.size()) * num_slabs > resident) return false;      // later work-groups go wherever one retires
    const uint32_t groups = (uint32_t(chunks.size()) + wpg - 1) / wpg;
    const uint32_t per_xcd = (groups + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd;
    const size_t span = size_t(per_xcd) * wpg;
    const uint32_t simds = cus_per_xcd * 4u;
    auto simd_of = [&](uint32_t pos, uint32_t y) {
        const uint32_t s = y * per_xcd + pos / wpg;
        return (s % cus_per_xcd) * 4u + (pos % wpg + s / cus_per_xcd) % 4u;
    };
    std::vector<uint4> dealt(chunks);
    uint64_t before = 0, after = 0;
    std::vector<uint64_t> load(simds);
    std::vector<uint32_t> order;
    std::vector<uint8_t> taken;
    for (uint32_t x = 0; x < cute_dev::kNumXcd; ++x) {
        const size_t b = std::min(chunks.size(), x * span), e = std::min(chunks.size(), (x + 1) * span);
        if (e <= b) continue;
        const uint32_t n = uint32_t(e - b);
        auto cost = [&](uint32_t i) { return uint64_t(chunks[b + i].y - chunks[b + i].x) + 2u; };
        std::fill(load.begin(), load.end(), 0);
        for (uint32_t i = 0; i < n; ++i)
            for (uint32_t y = 0; y < num_slabs; ++y) load[simd_of(i, y)] += cost(i);
        before = std::max(before, *std::max_element(load.begin(), load.end()));
        order.resize(n);
        for (uint32_t i = 0; i < n; ++i) order[i] = i;
        std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t c2) { return cost(a) > cost(c2); });
        std::fill(load.begin(), load.end(), 0);
        taken.assign(n, 0);
        for (uint32_t i : order) {
            uint32_t best = n;
            uint64_t best_peak = ~uint64_t(0);
            for (uint32_t pos = 0; pos < n; ++pos) {
                if (taken[pos]) continue;
                uint64_t peak = 0;
                for (uint32_t y = 0; y < num_slabs; ++y) peak = std::max(peak, load[simd_of(pos, y)]);
                if (peak < best_peak) { best_peak = peak; best = pos; }
                if (peak == 0) break;                                      // nothing beats an idle SIMD
            }
            taken[best] = 1;
            dealt[b + best] = chunks[b + i];
            for (uint32_t y = 0; y < num_slabs; ++y) load[simd_of(best, y)] += cost(i);
        }
        after = std::max(after, *std::max_element(load.begin(), load.end()));
    }
    if (!force && after * 100u > before * 97u) return false;
    chunks.swap(dealt);
    return true;
}

}  // namespace

extern "C" {

const char *cute_last_hip_error(void) { return g_hip_error.c_str(); }

int cute_device_info(int *num_cus, int *wave_size, char *arch_name, size_t arch_cap)
{
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    if (num_cus) *num_cus = c.num_cus;
    if (wave_size) *wave_size = c.wave_size;
    if (arch_name && arch_cap) std::snprintf(arch_name, arch_cap, "%s", c.arch.c_str());
    return CUTE_OK;
}

int cute_device_layout(int *num_xcds, int *cus_per_xcd, uint64_t *cache_bytes, int *whole_chip)
{
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    if (num_xcds) *num_xcds = c.num_xcds;
    if (cus_per_xcd) *cus_per_xcd = c.num_cus / c.num_xcds;
    if (cache_bytes) *cache_bytes = c.cache_bytes;
    if (whole_chip) *whole_chip = c.whole_chip ? 1 : 0;
    return CUTE_OK;
}

void cute_hrpb_dev_free(cute_hrpb_dev *d)
{
    if (!d) return;
    (void)hipFree(d->dHdr);
    (void)hipFree(d->dVals);
    (void)hipFree(d->dRowPtr);
    (void)hipFree(d->dCols);
    (void)hipFree(d->dCsrVals);
    (void)hipFree(d->dQRecs);
    (void)hipFree(d->dQVals);
    delete d;
}

uint64_t cute_hrpb_dev_bytes(const cute_hrpb_dev *d) { return d ? d->bytes : 0; }

int cute_hrpb_upload(const cute_hrpb_host *h, cute_hrpb_dev **out) { return cute_hrpb_upload_layout(h, 0, out); }

}  // extern "C"

namespace {

// ---- building the layouts on the device (kernels: build_kernels.hip.hpp) ----

struct DevBuf {                       // device memory that lives as long as a scope
    void *p = nullptr;
    DevBuf() = default;
    DevBuf(const DevBuf &) = delete;
    DevBuf &operator=(const DevBuf &) = delete;
    ~DevBuf() { if (p) (void)hipFree(p); }
    int alloc(uint64_t bytes)
    {
        HIP_TRY(hipMalloc(&p, std::max<uint64_t>(bytes, 16)));
        return CUTE_OK;
    }
    template <class T> T *as() const { return static_cast<T *>(p); }
};

inline dim3 grid_of(uint64_t n) { return dim3(uint32_t((n + cute_build::kThreads - 1) / cute_build::kThreads)); }

int check_launch(const char *what);

// Inclusive prefix sum of n uint32 values, in place, on the default stream.
int device_scan(uint32_t *data, uint64_t n)
{
    if (!n) return CUTE_OK;
    const uint64_t nb = (n + cute_build::kScanBlock - 1) / cute_build::kScanBlock;
    if (nb > 0x7fffffffull) return CUTE_ERR_SHAPE;
    if (nb == 1) {
        hipLaunchKernelGGL(cute_build::scan_block_apply, dim3(1), dim3(cute_build::kThreads), 0, nullptr, data, data, n,
                           static_cast<const uint32_t *>(nullptr));
        return check_launch("prefix sum");
    }
    DevBuf sums;
    int rc = sums.alloc(nb * sizeof(uint32_t));
    if (rc != CUTE_OK) return rc;
    hipLaunchKernelGGL(cute_build::scan_block_sums, dim3(uint32_t(nb)), dim3(cute_build::kThreads), 0, nullptr, data, n, sums.as<uint32_t>());
    rc = device_scan(sums.as<uint32_t>(), nb);
    if (rc != CUTE_OK) return rc;
    hipLaunchKernelGGL(cute_build::scan_block_apply, dim3(uint32_t(nb)), dim3(cute_build::kThreads), 0, nullptr, data, data, n,
                       sums.as<const uint32_t>());
    rc = check_launch("prefix sum");
    // (the block sums are freed when this scope ends; hipFree waits for the kernels that read them)
    return rc;
}

// Where every entry of the device CSR copy stands in the (column, row) order of its panel and of its strip,
// and the running count of distinct columns along both orders.  Checks that rows are sorted, duplicate-free
// and inside K.  With the two vectors given, also counts active columns per panel and list pairs per strip.
struct Census {
    DevBuf rowOf, posP, posS, DP, DS;
};

int device_census(const cute_hrpb_dev *d, Census &c, std::vector<uint32_t> *panelCols, std::vector<uint32_t> *stripPairs,
                  std::vector<uint32_t> *panelSpan = nullptr)
{
    const uint32_t nnz = d->nnz, P = d->P;
    if (panelCols) panelCols->assign(P, 0u);
    if (stripPairs) stripPairs->assign(size_t(P) * 4u, 0u);
    if (panelSpan) panelSpan->assign(P, 0u);
    if (!nnz) return CUTE_OK;
    const uint64_t bytes = uint64_t(nnz) * sizeof(uint32_t);
    int rc = c.rowOf.alloc(bytes);
    if (rc == CUTE_OK) rc = c.posP.alloc(bytes);
    if (rc == CUTE_OK) rc = c.posS.alloc(bytes);
    if (rc == CUTE_OK) rc = c.DP.alloc(bytes);
    if (rc == CUTE_OK) rc = c.DS.alloc(bytes);
    DevBuf err;
    if (rc == CUTE_OK) rc = err.alloc(sizeof(int));
    if (rc != CUTE_OK) return rc;
    HIP_TRY(hipMemset(err.p, 0, sizeof(int)));
    hipLaunchKernelGGL(cute_build::row_of_entries, grid_of(nnz), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCols, d->M,
                       d->K, nnz, c.rowOf.as<uint32_t>(), err.as<int>());
    int bad = 0;
    HIP_TRY(hipMemcpy(&bad, err.p, sizeof(int), hipMemcpyDeviceToHost));
    if (bad & cute_build::kErrRange) return CUTE_ERR_RANGE;
    if (bad & cute_build::kErrUnsorted) return CUTE_ERR_UNSORTED;
    hipLaunchKernelGGL(cute_build::entry_positions, grid_of(nnz), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCols,
                       c.rowOf.as<const uint32_t>(), nnz, c.posP.as<uint32_t>(), c.posS.as<uint32_t>(), c.DP.as<uint32_t>(),
                       c.DS.as<uint32_t>());
    rc = check_launch("entry positions");
    if (rc == CUTE_OK) rc = device_scan(c.DP.as<uint32_t>(), nnz);
    if (rc == CUTE_OK) rc = device_scan(c.DS.as<uint32_t>(), nnz);
    if (rc != CUTE_OK || !panelCols || !stripPairs) return rc;
    DevBuf pc, sp, span;
    rc = pc.alloc(uint64_t(P) * 4u);
    if (rc == CUTE_OK) rc = sp.alloc(uint64_t(P) * 16u);
    if (rc == CUTE_OK) rc = span.alloc(uint64_t(P) * 4u);
    if (rc != CUTE_OK) return rc;
    hipLaunchKernelGGL(cute_build::count_columns, grid_of(uint64_t(P) * 4u), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCols,
                       c.DP.as<const uint32_t>(), c.DS.as<const uint32_t>(), P, pc.as<uint32_t>(), sp.as<uint32_t>(), span.as<uint32_t>());
    HIP_TRY(hipMemcpy(panelCols->data(), pc.p, uint64_t(P) * 4u, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(stripPairs->data(), sp.p, uint64_t(P) * 16u, hipMemcpyDeviceToHost));
    if (panelSpan) HIP_TRY(hipMemcpy(panelSpan->data(), span.p, uint64_t(P) * 4u, hipMemcpyDeviceToHost));
    return CUTE_OK;
}

// Brick tiles from the device CSR copy: the arrays cute_hrpb_retile makes on the host, word for word.
int build_bricks_on_device(cute_hrpb_dev *d, const Census &c)
{
    const uint64_t hdr_words = uint64_t(d->nb) * CUTE_TILED_HDR_WORDS, num_vals = uint64_t(d->nnz) + 64u;
    uint32_t *hdr = nullptr, *brp = nullptr, *pcols = nullptr;
    float *vals = nullptr;
    DevBuf hdr_buf, vals_buf, brp_buf, pc_buf;
    int rc = hdr_buf.alloc(hdr_words * 4u);
    if (rc == CUTE_OK) rc = vals_buf.alloc(num_vals * 4u);
    if (rc == CUTE_OK) rc = brp_buf.alloc((uint64_t(d->P) + 1u) * 4u);
    if (rc == CUTE_OK) rc = pc_buf.alloc(uint64_t(d->P) * 4u);
    if (rc != CUTE_OK) return rc;
    hdr = hdr_buf.as<uint32_t>(); vals = vals_buf.as<float>(); brp = brp_buf.as<uint32_t>(); pcols = pc_buf.as<uint32_t>();
    HIP_TRY(hipMemset(hdr, 0, std::max<uint64_t>(hdr_words * 4u, 4u)));
    HIP_TRY(hipMemset(vals + d->nnz, 0, 64u * sizeof(float)));          // one wavefront of zeros behind the values
    HIP_TRY(hipMemcpy(brp, d->brp.data(), (uint64_t(d->P) + 1u) * 4u, hipMemcpyHostToDevice));
    if (d->P) HIP_TRY(hipMemcpy(pcols, d->panelCols.data(), uint64_t(d->P) * 4u, hipMemcpyHostToDevice));
    if (d->nnz) {
        hipLaunchKernelGGL(cute_build::brick_scatter, grid_of(d->nnz), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCols,
                           d->dCsrVals, c.rowOf.as<const uint32_t>(), c.posP.as<const uint32_t>(), c.DP.as<const uint32_t>(), brp,
                           d->nnz, hdr, vals);
        hipLaunchKernelGGL(cute_build::brick_finish, grid_of(d->nb), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, brp, pcols,
                           d->P, d->nb, hdr);
        rc = check_launch("brick tiles");
        if (rc != CUTE_OK) return rc;
    }
    HIP_TRY(hipDeviceSynchronize());
    d->dHdr = hdr; hdr_buf.p = nullptr;
    d->dVals = vals; vals_buf.p = nullptr;
    d->bytes += hdr_words * 4u + num_vals * 4u;
    d->haveBricks = true;
    return CUTE_OK;
}

// Quad lists (in the layout the census chose) from the device CSR copy: the arrays cute_quad_pack makes.
int build_quads_on_device(cute_hrpb_dev *d, const Census &c)
{
    const uint64_t G = d->numGroups;
    const uint32_t U = uint32_t(d->qgp.size() - 1);
    const bool strips = d->quadRows == 4;
    DevBuf recs_buf, qgp_buf, sp_buf, counts_buf, vals_buf;
    int rc = recs_buf.alloc(G * CUTE_QUAD_RECORD_WORDS * 4u);
    if (rc == CUTE_OK) rc = qgp_buf.alloc(d->qgp.size() * 4u);
    if (rc == CUTE_OK) rc = sp_buf.alloc(d->stripPairs.size() * 4u);
    if (rc == CUTE_OK) rc = counts_buf.alloc(G * 4u);
    if (rc != CUTE_OK) return rc;
    uint32_t *recs = recs_buf.as<uint32_t>(), *qgp = qgp_buf.as<uint32_t>(), *sp = sp_buf.as<uint32_t>(), *counts = counts_buf.as<uint32_t>();
    HIP_TRY(hipMemset(recs, 0, std::max<uint64_t>(G * CUTE_QUAD_RECORD_WORDS * 4u, 4u)));
    HIP_TRY(hipMemcpy(qgp, d->qgp.data(), d->qgp.size() * 4u, hipMemcpyHostToDevice));
    if (!d->stripPairs.empty()) HIP_TRY(hipMemcpy(sp, d->stripPairs.data(), d->stripPairs.size() * 4u, hipMemcpyHostToDevice));
    uint32_t stored = 0;
    if (G) {
#define CUTE_BUILD_QUADS(S)                                                                                                          \
    hipLaunchKernelGGL(cute_build::quad_scatter<S>, grid_of(d->nnz), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCols,     \
                       d->dCsrVals, c.rowOf.as<const uint32_t>(), c.posS.as<const uint32_t>(), c.DS.as<const uint32_t>(), qgp, d->nnz, \
                       recs);                                                                                                        \
    hipLaunchKernelGGL(cute_build::quad_groups<S>, grid_of(G), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCols, qgp, U, sp, \
                       uint32_t(G), recs, counts)
        if (strips) { CUTE_BUILD_QUADS(true); } else { CUTE_BUILD_QUADS(false); }
#undef CUTE_BUILD_QUADS
        rc = check_launch("quad lists");
        if (rc == CUTE_OK) rc = device_scan(counts, G);
        if (rc != CUTE_OK) return rc;
        hipLaunchKernelGGL(cute_build::quad_first_values, grid_of(G), dim3(cute_build::kThreads), 0, nullptr, counts, uint32_t(G), recs);
        HIP_TRY(hipMemcpy(&stored, counts + (G - 1u), sizeof(uint32_t), hipMemcpyDeviceToHost));
    }
    rc = vals_buf.alloc((uint64_t(stored) + 64u) * 4u);
    if (rc != CUTE_OK) return rc;
    float *packed = vals_buf.as<float>();
    HIP_TRY(hipMemset(packed, 0, (uint64_t(stored) + 64u) * 4u));
    if (G && d->nnz) {
        if (strips)
            hipLaunchKernelGGL(cute_build::quad_values<true>, grid_of(d->nnz), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCsrVals,
                               c.rowOf.as<const uint32_t>(), c.posS.as<const uint32_t>(), c.DS.as<const uint32_t>(), qgp, d->nnz, recs, packed);
        else
            hipLaunchKernelGGL(cute_build::quad_values<false>, grid_of(d->nnz), dim3(cute_build::kThreads), 0, nullptr, d->dRowPtr, d->dCsrVals,
                               c.rowOf.as<const uint32_t>(), c.posS.as<const uint32_t>(), c.DS.as<const uint32_t>(), qgp, d->nnz, recs, packed);
        rc = check_launch("quad values");
        if (rc != CUTE_OK) return rc;
    }
    HIP_TRY(hipDeviceSynchronize());
    d->numQuadVals = stored;
    d->dQRecs = recs; recs_buf.p = nullptr;
    d->dQVals = packed; vals_buf.p = nullptr;
    d->bytes += G * CUTE_QUAD_RECORD_WORDS * 4u + (uint64_t(stored) + 64u) * 4u;
    d->haveQuads = true;
    return CUTE_OK;
}

// A layout the upload did not build: made on the device from the device copy of the CSR arrays (the host
// arrays the format borrowed may be gone by now).  which: 1 brick tiles, 2 quad lists.
int ensure_layout(cute_hrpb_dev *d, int which)
{
    std::lock_guard<std::mutex> guard(d->lock);
    if (which == 1 ? d->haveBricks : d->haveQuads) return CUTE_OK;
    Census c;
    int rc = device_census(d, c, nullptr, nullptr);
    if (rc != CUTE_OK) return rc;
    return which == 1 ? build_bricks_on_device(d, c) : build_quads_on_device(d, c);
}

// Group counts of the quad lists from the list length of every strip; picks lockstep lists unless they would
// be mostly padding (a few very long rows stretch the lists of their panel neighbours): then one list per strip.
int finish_quad_census(cute_hrpb_dev *d, std::vector<uint32_t> &strip_pairs, int quad_layout)
{
    const uint32_t S = d->M / 4;
    uint64_t pairs = 0, lock_groups = 0;
    for (uint32_t p = 0; p < d->P; ++p) {
        uint32_t longest = 0;
        for (uint32_t l = 0; l < 4; ++l) { longest = std::max(longest, strip_pairs[4 * p + l]); pairs += strip_pairs[4 * p + l]; }
        lock_groups += (longest + 3) / 4;
    }
    if (quad_layout == 0) quad_layout = (lock_groups && double(pairs) < 0.6 * 16.0 * double(lock_groups)) ? 2 : 1;
    d->quadRows = quad_layout == 2 ? 4u : CUTE_TM;
    d->quadPairs = pairs;
    const uint32_t per_unit = d->quadRows / 4, U = S / per_unit;
    d->qgp.assign(size_t(U) + 1, 0u);
    uint64_t groups = 0;
    for (uint32_t u = 0; u < U; ++u) {
        uint32_t longest = 0;
        for (uint32_t l = 0; l < per_unit; ++l) longest = std::max(longest, strip_pairs[u * per_unit + l]);
        groups += per_unit == 4 ? (longest + 3) / 4 : (longest + 15) / 16;
        if (groups > 0xffffffffull / 64) return CUTE_ERR_SHAPE;
        d->qgp[u + 1] = uint32_t(groups);
    }
    d->numGroups = groups;
    d->stripPairs.swap(strip_pairs);
    return CUTE_OK;
}

// Which MFMA layout would the planner's default rules use for this matrix (see cute_spmm_plan_create)?
// 0: none (every panel would go to the row kernel), 1 brick tiles, 2 quad lists.
int default_layout(const cute_hrpb_dev *d, uint64_t cache_bytes)
{
    const uint32_t lists = d->quadRows == 4 ? 4u : 1u;
    uint64_t slots = 0, bricks = 0, blocks = 0;
    for (uint32_t q = 0; q < d->P; ++q) {
        if (d->brp[q + 1] == d->brp[q]) continue;
        const uint32_t list_slots = (d->qgp[(q + 1) * lists] - d->qgp[q * lists]) * 16u;
        const uint32_t fetches = std::max(d->panelCols[q], list_slots);
        if (float(d->panelNnz[q]) < kMinReuse * float(fetches) && d->panelMaxRow[q] <= kMaxRowForRows) continue;   // row kernel
        slots += list_slots;
        bricks += (d->panelCols[q] + 3u) / 4u;
        blocks += d->brp[q + 1] - d->brp[q];
    }
    if (!bricks) return 0;
    // (the width is not known yet: 128 columns stand in for it)
    return choose_mfma_shape(slots, bricks, blocks, uint64_t(d->K) + d->M, d->nnz, 128u, 0u, cache_bytes);
}

// The common tail of both uploads.  d holds the device copy of the CSR arrays, rowPtr is a host copy of the row
// pointers (checked: ascending from 0 to nnz).  Counts active columns per panel and list pairs per strip on the
// device, derives the planner's per-panel statistics, and builds the one MFMA layout the planner's default
// rules would use for this matrix (none when every panel would go to the row kernel).
int finish_upload(cute_hrpb_dev *d, const uint32_t *rowPtr, int quad_layout, const DeviceContext &c)
{
    Census cen;
    std::vector<uint32_t> strip_pairs;
    int rc = device_census(d, cen, &d->panelCols, &strip_pairs, &d->panelSpan);
    if (rc != CUTE_OK) return rc;
    d->brp.assign(size_t(d->P) + 1, 0u);
    d->panelNnz.resize(d->P);
    d->panelMaxRow.resize(d->P);
    uint64_t blocks = 0;
    for (uint32_t p = 0; p < d->P; ++p) {
        d->panelNnz[p] = rowPtr[(p + 1) * CUTE_TM] - rowPtr[p * CUTE_TM];
        uint32_t longest = 0;
        for (uint32_t r = p * CUTE_TM; r < (p + 1) * CUTE_TM; ++r) longest = std::max(longest, rowPtr[r + 1] - rowPtr[r]);
        d->panelMaxRow[p] = longest;
        blocks += (d->panelCols[p] + CUTE_TK - 1) / CUTE_TK;
        if (blocks > 0xffffffffull / CUTE_TILED_HDR_WORDS) return CUTE_ERR_SHAPE;
        d->brp[p + 1] = uint32_t(blocks);
    }
    d->nb = uint32_t(blocks);
    rc = finish_quad_census(d, strip_pairs, quad_layout);
    if (rc != CUTE_OK) return rc;
    const int which = default_layout(d, c.cache_bytes);
    if (which == 2) rc = build_quads_on_device(d, cen);
    else if (which == 1) rc = build_bricks_on_device(d, cen);
    return rc;
}

// Tables of a hub plan: the hub_rows most referenced columns of the quad records (ties: the lower column) get
// the slots 0.. of the LDS table; the plan keeps their column ids in slot order and its own copy of the records
// in which those columns name their slot.
int make_hub_tables(cute_spmm_plan *p, const cute_hrpb_dev *d, uint32_t hub_rows)
{
    const uint64_t G = d->numGroups;
    DevBuf counts, slots;
    int rc = counts.alloc(uint64_t(d->K) * 4u);
    if (rc == CUTE_OK) rc = slots.alloc(uint64_t(d->K) * 4u);
    if (rc != CUTE_OK) return rc;
    HIP_TRY(hipMemset(counts.p, 0, uint64_t(d->K) * 4u));
    hipLaunchKernelGGL(cute_build::count_record_columns, grid_of(G * 16u), dim3(cute_build::kThreads), 0, nullptr, d->dQRecs, G,
                       counts.as<uint32_t>());
    std::vector<uint32_t> cnt(d->K), order(d->K), slot_of(d->K, ~0u);
    HIP_TRY(hipMemcpy(cnt.data(), counts.p, uint64_t(d->K) * 4u, hipMemcpyDeviceToHost));
    for (uint32_t k = 0; k < d->K; ++k) order[k] = k;
    std::partial_sort(order.begin(), order.begin() + hub_rows, order.end(),
                      [&](uint32_t a, uint32_t b) { return cnt[a] != cnt[b] ? cnt[a] > cnt[b] : a < b; });
    uint32_t used = 0;
    while (used < hub_rows && cnt[order[used]] > 1u) ++used;            // a row fetched once gains nothing from LDS
    if (!used) return CUTE_OK;
    for (uint32_t h = 0; h < used; ++h) slot_of[order[h]] = h;
    HIP_TRY(hipMemcpy(slots.p, slot_of.data(), uint64_t(d->K) * 4u, hipMemcpyHostToDevice));
    rc = upload(&p->dHubRows, order.data(), used);
    if (rc != CUTE_OK) return rc;
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&p->dHubRecs), std::max<uint64_t>(G * CUTE_QUAD_RECORD_WORDS * 4u, 16u)));
    hipLaunchKernelGGL(cute_build::mark_hub_columns, grid_of(G * CUTE_QUAD_RECORD_WORDS), dim3(cute_build::kThreads), 0, nullptr,
                       d->dQRecs, G, slots.as<const uint32_t>(), uint32_t(cute_dev::kHubFlag), p->dHubRecs);
    rc = check_launch("hub records");
    if (rc != CUTE_OK) return rc;
    HIP_TRY(hipDeviceSynchronize());
    p->numHub = used;
    return CUTE_OK;
}

}  // namespace

extern "C" {

int cute_hrpb_upload_layout(const cute_hrpb_host *h, int quad_layout, cute_hrpb_dev **out)
{
    if (!h || !out || !h->rowPtr || quad_layout < 0 || quad_layout > 2) return CUTE_ERR_ARG;
    *out = nullptr;
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    if (h->M == 0 || h->M % CUTE_TM || h->K % CUTE_TK) return CUTE_ERR_SHAPE;
    cute_hrpb_dev *d = new cute_hrpb_dev;
    d->M = h->M;
    d->K = h->K;
    d->nnz = h->nnz;
    d->P = h->numRowPanels;
    d->numVals = h->nnz;                     // the brick tiles store every entry of the matrix once
    int rc = upload(&d->dRowPtr, h->rowPtr, uint64_t(h->M) + 1);
    if (rc == CUTE_OK) rc = upload(&d->dCols, h->cols, h->nnz);
    if (rc == CUTE_OK) rc = upload(&d->dCsrVals, h->vals, h->nnz);
    d->bytes = (uint64_t(h->M) + 1) * 4 + uint64_t(h->nnz) * 8;
    if (rc == CUTE_OK) rc = finish_upload(d, h->rowPtr, quad_layout, c);
    // the device counted the active columns itself: it must have found the blocks the canonical format has
    if (rc == CUTE_OK && (d->nb != h->numBlocks || std::memcmp(d->brp.data(), h->blockedRowPtr, d->brp.size() * sizeof(uint32_t)) != 0))
        rc = CUTE_ERR_FORMAT;
    if (rc != CUTE_OK) { cute_hrpb_dev_free(d); return rc; }
    *out = d;
    return CUTE_OK;
}

// The device-side counterpart of HRPB::HRPB + DATASTRUCT (data.cu:80-335, timed at run.cu:17-20) for a CSR
// matrix that already lives on the device: the handle keeps its own copy of the three arrays (device to
// device), the layouts are built by kernels, and only per-panel and per-strip counts (and the row pointers,
// for the planner's per-panel statistics) travel to the host.
int cute_hrpb_upload_device_csr(uint32_t M, uint32_t K, uint32_t nnz, const uint32_t *dRowPtr, const uint32_t *dCols,
                                const float *dVals, int quad_layout, cute_hrpb_dev **out)
{
    if (!out || !dRowPtr || (nnz && (!dCols || !dVals)) || quad_layout < 0 || quad_layout > 2) return CUTE_ERR_ARG;
    *out = nullptr;
    if (M == 0 || K == 0 || M % CUTE_TM || K % CUTE_TK) return CUTE_ERR_SHAPE;
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    // the row pointers come to the host first: everything on the device indexes through them
    std::vector<uint32_t> rowPtr(size_t(M) + 1);
    HIP_TRY(hipMemcpy(rowPtr.data(), dRowPtr, rowPtr.size() * sizeof(uint32_t), hipMemcpyDeviceToHost));
    if (rowPtr[0] != 0 || rowPtr[M] != nnz) return CUTE_ERR_RANGE;
    for (uint32_t r = 0; r < M; ++r)
        if (rowPtr[r + 1] < rowPtr[r]) return CUTE_ERR_RANGE;
    cute_hrpb_dev *d = new cute_hrpb_dev;
    d->M = M; d->K = K; d->nnz = nnz; d->P = M / CUTE_TM;
    d->numVals = nnz;
    auto clone = [&](auto **dst, const auto *src, uint64_t count) -> int {
        HIP_TRY(hipMalloc(reinterpret_cast<void **>(dst), std::max<uint64_t>(count, 1) * 4u));
        if (count) HIP_TRY(hipMemcpy(*dst, src, count * 4u, hipMemcpyDeviceToDevice));
        return CUTE_OK;
    };
    int rc = clone(&d->dRowPtr, dRowPtr, uint64_t(M) + 1);
    if (rc == CUTE_OK) rc = clone(&d->dCols, dCols, nnz);
    if (rc == CUTE_OK) rc = clone(&d->dCsrVals, dVals, nnz);
    d->bytes = (uint64_t(M) + 1) * 4 + uint64_t(nnz) * 8;
    if (rc == CUTE_OK) rc = finish_upload(d, rowPtr.data(), quad_layout, c);
    if (rc != CUTE_OK) { cute_hrpb_dev_free(d); return rc; }
    *out = d;
    return CUTE_OK;
}

// Sizes and host copies of what a device handle holds, for inspection and tests.  Layouts that were not built
// have size 0; pass nullptr for arrays that are not wanted.
int cute_hrpb_dev_layout_sizes(const cute_hrpb_dev *d, uint32_t *numBlocks, uint64_t *numTileVals, uint64_t *numGroups,
                               uint64_t *numQuadVals, uint32_t *rowsPerList)
{
    if (!d) return CUTE_ERR_ARG;
    if (numBlocks) *numBlocks = d->haveBricks ? d->nb : 0u;
    if (numTileVals) *numTileVals = d->haveBricks ? d->numVals : 0u;
    if (numGroups) *numGroups = d->haveQuads ? d->numGroups : 0u;
    if (numQuadVals) *numQuadVals = d->haveQuads ? d->numQuadVals : 0u;
    if (rowsPerList) *rowsPerList = d->quadRows;
    return CUTE_OK;
}

int cute_hrpb_dev_read_layouts(const cute_hrpb_dev *d, uint32_t *blockedRowPtr, uint32_t *hdr, float *tileVals, uint32_t *groupPtr,
                               uint32_t *recs, float *quadVals)
{
    if (!d) return CUTE_ERR_ARG;
    if (blockedRowPtr) std::memcpy(blockedRowPtr, d->brp.data(), d->brp.size() * sizeof(uint32_t));
    if (groupPtr) std::memcpy(groupPtr, d->qgp.data(), d->qgp.size() * sizeof(uint32_t));
    if (d->haveBricks) {
        if (hdr && d->nb) HIP_TRY(hipMemcpy(hdr, d->dHdr, uint64_t(d->nb) * CUTE_TILED_HDR_WORDS * 4u, hipMemcpyDeviceToHost));
        if (tileVals && d->numVals) HIP_TRY(hipMemcpy(tileVals, d->dVals, d->numVals * 4u, hipMemcpyDeviceToHost));
    }
    if (d->haveQuads) {
        if (recs && d->numGroups) HIP_TRY(hipMemcpy(recs, d->dQRecs, d->numGroups * CUTE_QUAD_RECORD_WORDS * 4u, hipMemcpyDeviceToHost));
        if (quadVals && d->numQuadVals) HIP_TRY(hipMemcpy(quadVals, d->dQVals, d->numQuadVals * 4u, hipMemcpyDeviceToHost));
    }
    return CUTE_OK;
}

int cute_hrpb_dev_csr(const cute_hrpb_dev *d, const uint32_t **dRowPtr, const uint32_t **dCols, const float **dVals)
{
    if (!d) return CUTE_ERR_ARG;
    if (dRowPtr) *dRowPtr = d->dRowPtr;
    if (dCols) *dCols = d->dCols;
    if (dVals) *dVals = d->dCsrVals;
    return CUTE_OK;
}

void cute_spmm_plan_free(cute_spmm_plan *p)
{
    if (!p) return;
    (void)hipFree(p->dChunks);
    (void)hipFree(p->dHeads);
    (void)hipFree(p->dHubRows);
    (void)hipFree(p->dHubRecs);
    (void)hipFree(p->dFixups);
    (void)hipFree(p->dPartials);
    (void)hipFree(p->dRowList);
    delete p;
}

int cute_spmm_plan_info(const cute_spmm_plan *p, cute_plan_info *out)
{
    if (!p || !out) return CUTE_ERR_ARG;
    *out = p->info;
    return CUTE_OK;
}

// Replaces SPMM_TC's constructor chain (spmm.cu:276-822).  The per-N launch shapes of
// spmm.cu:11-101 and the occupancy table of spmm.cu:290-690 describe NVIDIA parts; here
// the shape follows from wave64 MFMA tiles (16 lanes x VEC columns per group) and the slot
// count from the CU count of the device.
int cute_spmm_plan_create(cute_hrpb_dev *d, uint32_t N, const cute_tunables *tn, cute_spmm_plan **out)
{
    if (!d || !out) return CUTE_ERR_ARG;
    *out = nullptr;
    if (N == 0) return CUTE_ERR_SHAPE;
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    cute_tunables t{};
    if (tn) t = *tn;
    if (t.path < CUTE_PATH_AUTO || t.path > CUTE_PATH_ROWS) return CUTE_ERR_ARG;
    if (t.precision != CUTE_PREC_FP32 && t.precision != CUTE_PREC_BF16X3) return CUTE_ERR_ARG;
    const float min_reuse = t.min_reuse > 0.0f ? t.min_reuse : kMinReuse;
    const uint32_t max_row_for_rows = t.max_row_nnz ? t.max_row_nnz : kMaxRowForRows;
    // An MFMA work item always spans 64 output columns; when N is narrower the row kernel wastes
    // less, so the reuse a panel must offer to earn the MFMA kernel grows (measured on N = 8..32).
    const float reuse_bar = N <= 32 ? std::min(3.0f, min_reuse * 48.0f / float(N)) : min_reuse;
    // Wide products of large matrices: the row kernel walks three dependent round trips per row (row pointers,
    // entries, B rows), the quad kernel streams its lists two groups ahead, and with 256 columns or more and a launch
    // several times the size of the device that depth counts for more than reuse: on 50 000 rows of 7 entries at
    // random columns, N = 512, the quad kernel takes 93 us against 116; ncvxbqp1, mk12-b3, delaunay_n16 of the
    // reference's matrices gain 10-20 % the same way.  There the bar drops to "the lists need no more fetches than the
    // panel has entries" (matrices whose short lists would be mostly padding -- cat_ears_4_4, Wordnet3 -- stay with
    // the row kernel, which is 20 % ahead on them).
    // ... provided the panel's B rows cannot come out of an L2 anyway: a banded matrix, whose panels read a window of B
    // that the L2s hold (the banded benchmark matrix: 4 112 columns), is bound by the L2-to-L1 gather rate, where the row
    // kernel's 16 bytes per lane beat the quad kernel's 4 (1 736 against 2 046 us), and keeps the usual bar.
    const bool wide_and_large = t.min_reuse <= 0.0f && N >= 256u &&
                                uint64_t(d->M) * ((N + 255u) / 256u) >= 4ull * uint64_t(c.num_cus) * 32u;

    cute_spmm_plan *p = new cute_spmm_plan;
    p->d = d;
    // classify panels
    std::vector<uint8_t> to_rows(d->P, 0);
    // panels that go to the MFMA kernel for another reason than their reuse (below); the choice of the MFMA shape is
    // made on the panels that earned it
    std::vector<uint8_t> joined(d->P, 0);
    // The row kernel gives a row N / VEC lanes; up to N = 128 several rows share a wavefront, which then takes as long
    // as its longest row.  A panel whose longest row is more than twice its mean row (and longer than two batches of
    // eight entries) keeps its wavefronts waiting for that one row, and the MFMA kernel, which walks the panel's
    // columns whatever row they belong to, is ahead although the reuse is low: on the reference's matrices with
    // long-tailed rows (jan99jac*, de2010, ri2010, Wordnet3, bayer04, ted_B: 99th percentile of the row lengths 3-6 times
    // the mean) 25-35 % at N = 16 and 32, geomean over the 43 matrices against the best single kernel 1.18 -> 1.10
    // (N = 16), 1.10 -> 1.04 (N = 32), 1.07 -> 1.03 (N = 128).  With one row per wavefront (N >= 256) the same move
    // loses (HEP-th-new, N = 512: 60 -> 68 us), so it is not made there.
    const uint32_t row_lane_width = (N % 4 == 0) ? 4u : (N % 2 == 0) ? 2u : 1u;      // floats per lane of the row kernel
    const bool rows_share_a_wavefront = t.max_row_nnz == 0 && (N + row_lane_width - 1u) / row_lane_width < 64u;
    uint32_t n_brick = 0, n_rows = 0, n_empty = 0;
    for (uint32_t q = 0; q < d->P; ++q) {
        const uint32_t nblk = d->brp[q + 1] - d->brp[q];
        bool rows;
        if (nblk == 0) { rows = true; n_empty++; }
        else if (t.path == CUTE_PATH_BRICK) rows = false;
        else if (t.path == CUTE_PATH_ROWS) rows = true;
        else {
            // Row kernel when a B row fetched by the MFMA side serves hardly more than one nonzero of the
            // panel (the matrix cores then buy nothing) -- unless a row is so long that one lane group
            // would serialise it: the brick kernel cuts long panels into balanced chunks.
            // what the MFMA side would fetch for this panel: one B row per list slot of the quad
            // lists (pairs plus padding), which is at least one per active column
            const uint32_t lists = d->quadRows == 4 ? 4u : 1u;
            const uint32_t fetches = std::max(d->panelCols[q], (d->qgp[(q + 1) * lists] - d->qgp[q * lists]) * 16u);
            const float bar = (wide_and_large && uint64_t(d->panelSpan[q]) * N * sizeof(float) > kWideWindowBytes) ? kWideReuse : reuse_bar;
            rows = float(d->panelNnz[q]) < bar * float(fetches) && d->panelMaxRow[q] <= max_row_for_rows;
            if (rows && rows_share_a_wavefront && d->panelMaxRow[q] > kUnevenRowFloor &&
                uint64_t(d->panelMaxRow[q]) * CUTE_TM > uint64_t(kUnevenRowRatio) * d->panelNnz[q]) {
                rows = false;
                joined[q] = 1;
            }
        }
        to_rows[q] = rows;
        if (nblk) (rows ? n_rows : n_brick)++;
    }
    // A handful of MFMA panels among row-kernel panels (the boundary panels of a stencil at N = 32: 64 of 16 384) would
    // turn the launch into the fused kernel for their sake, which costs the row blocks more than those panels gain
    // (9-point stencil of 512 x 512 points, N = 32: 29.0 us against 24.4 with every panel on the row kernel): when
    // the MFMA panels hold less than 2 % of the entries and none of them has a row too long for a lane group,
    // they go to the row kernel as well.
    // The same the other way round: a few row-kernel panels among MFMA panels cost a second launch or the fused
    // kernel (FEM benchmark matrix, 53 of 3 000 panels: N = 8 21.2 us against 11.0 with every panel on the brick
    // kernel, N = 16 12.3 against 10.7, N = 24 16.7 against 14.0); below 2 % of the entries they join the others.
    if (t.path == CUTE_PATH_AUTO && n_brick && n_rows) {
        uint64_t nnz_mfma = 0;
        bool movable = true;
        for (uint32_t q = 0; q < d->P; ++q)
            if (!to_rows[q]) {
                nnz_mfma += d->panelNnz[q];
                movable = movable && d->panelMaxRow[q] <= max_row_for_rows;
            }
        if (movable && nnz_mfma * 50u < uint64_t(d->nnz)) {
            std::fill(to_rows.begin(), to_rows.end(), uint8_t(1));
            n_rows += n_brick;
            n_brick = 0;
        } else if ((uint64_t(d->nnz) - nnz_mfma) * 50u < uint64_t(d->nnz)) {
            for (uint32_t q = 0; q < d->P; ++q)
                if (to_rows[q] && d->brp[q + 1] != d->brp[q]) { to_rows[q] = 0; joined[q] = 1; }   // (empty panels stay: the row kernel zeroes their rows)
            n_brick += n_rows;
            n_rows = 0;
        }
    }

    // brick kernel shape
    p->vec = (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
    p->rows_vec = p->vec;
    // a brick work item spans 16*VEC columns: for narrow N take the narrowest tile that still covers N
    while (p->vec > 1 && 8u * uint32_t(p->vec) >= N) p->vec /= 2;
    p->ng = (p->vec == 4 && N >= 128) ? 2 : 1;   // two column groups per lane pay off from 128 columns on (measured)
    // row kernel shape: lanes per row = smallest power of two covering N/VEC, at most 64
    {
        uint32_t need = (N + p->rows_vec - 1) / p->rows_vec, logl = 0;
        while ((1u << logl) < need && logl < 6) ++logl;
        p->rows_logl = int(logl);
        const uint32_t w = (1u << logl) * p->rows_vec;
        p->rows_slabs = (N + w - 1) / w;
    }
    // A mixed plan is one launch, and the two-group brick kernel holds only four wavefronts per SIMD: when its
    // work-groups and the row blocks together exceed that, the row blocks queue behind each other and the launch
    // takes as long as the two parts one after the other (bcsstk18, N = 128: 11.8 us against 5.1 + 6.5).  One
    // column group per lane halves the registers and doubles the resident wavefronts; the same when the row blocks
    // are the larger part of the launch anyway (ted_B, N = 128).
    bool ng_for_mixed = false;
    // (not when B and C come from HBM: there the wider row pieces of two column groups count for more)
    if (t.operand_residency > 2) { delete p; return CUTE_ERR_ARG; }
    const bool beyond_cache = t.operand_residency ? t.operand_residency == 1
                                                  : (uint64_t(d->K) + d->M) * N * sizeof(float) > c.cache_bytes;
    if (p->ng == 2 && t.brick_groups == 0 && n_brick && n_rows && !beyond_cache) {
        const uint64_t row_blocks = (uint64_t(n_rows) * CUTE_TM * p->rows_slabs + (256u >> p->rows_logl) - 1) / (256u >> p->rows_logl);
        const uint64_t groups = (uint64_t(n_brick) * ((N + 127u) / 128u) + cute_dev::kWavesPerGroup - 1) / cute_dev::kWavesPerGroup;
        if (row_blocks + groups > uint64_t(c.num_cus) * 4u || row_blocks >= groups) { p->ng = 1; ng_for_mixed = true; }
    }
    if (t.brick_groups == 1 || (t.brick_groups == 2 && p->vec == 4)) p->ng = int(t.brick_groups);
    if (t.pipeline > 2) { delete p; return CUTE_ERR_ARG; }
    // the rolling variant addresses B and the values with 32-bit byte offsets (24 x 24-bit product)
    const bool offsets_fit = cute_offsets_fit(d->M, d->K, N, d->numVals, 0) == 1;
    p->pipeline = t.pipeline ? int(t.pipeline) : 1;
    if (p->pipeline == 1 && !offsets_fit) p->pipeline = 2;
    if (t.mfma_shape > 2) { delete p; return CUTE_ERR_ARG; }
    if (t.mfma_shape) p->shape = int(t.mfma_shape);
    else if (t.precision == CUTE_PREC_BF16X3) p->shape = 1;      // the reduced-precision kernel works on the brick tiles
    else {
        // A 16x4 brick costs the same matrix time however few nonzeros it holds; the quad lists
        // only pay for occupied (4-row group, column) pairs but fetch a B row once per row group
        // instead of once per panel, and pad their lists.  Measured break-even on the benchmark
        // matrices and on the reference's 43: about 8 list slots (pairs plus padding) per brick.
        const uint32_t lists = d->quadRows == 4 ? 4u : 1u;     // list units per panel
        uint64_t slots = 0, bricks = 0, blocks = 0;
        for (uint32_t q = 0; q < d->P; ++q)
            if (!to_rows[q] && !joined[q]) {
                slots += uint64_t(d->qgp[(q + 1) * lists] - d->qgp[q * lists]) * 16u;
                bricks += (d->panelCols[q] + 3u) / 4u;
                blocks += d->brp[q + 1] - d->brp[q];
            }
        p->shape = choose_mfma_shape(slots, bricks, blocks, uint64_t(d->K) + d->M, d->nnz, N, t.operand_residency, c.cache_bytes);
    }
    if (p->shape == 2 && !(offsets_fit && (d->numQuadVals + 64u) * 4u <= 0xffffffffull)) p->shape = 1;
    // bf16x3 exists for the rolling brick kernel with four columns per lane; any other shape computes in fp32
    p->bf16x3 = t.precision == CUTE_PREC_BF16X3 && p->shape == 1 && p->pipeline == 1 && p->vec == 4;
    // The chunk list depends on the MFMA kernel (its work units are blocks or list groups).  It is built,
    // and if the partial tiles of the cut panels then turn out to be more rows than the fast kernels'
    // 24-bit row operand can address, built once more for the pipelined brick kernel, whose stores use
    // 64-bit offsets.
    uint32_t slab = 0, num_slabs = 0, upp = 1, slots = 0, n_pieces = 0;
    std::vector<uint4> chunks, fixups;
    for (int attempt = 0;; ++attempt) {
        slab = p->shape == 2 ? 64u : 16u * p->vec * p->ng;   // the quad kernel: one column per lane
        num_slabs = (N + slab - 1) / slab;
        if (num_slabs > 65535u) { delete p; return CUTE_ERR_ARG; }   // slabs are the y dimension of the launch

        // chunk list for the brick kernel.  With t.slots set, the reference arithmetic
        // (spmm.cu:776-812) decides which panels are cut; its default there would cut every panel
        // that is one block above the (floored) mean as soon as the device holds all work items
        // at once, which is the normal case on 256 CUs.  The default policy therefore cuts only
        // outliers: a panel is split when it is more than twice as long as the per-item share
        // of the whole job (and at least 8 blocks), into pieces of about that share.
        // work units along a panel: 16-column blocks for the brick kernel, groups for the quad kernel
        const std::vector<uint32_t> &unit = p->shape == 2 ? d->qgp : d->brp;
        // units per panel: 4 when the quad lists are kept per 4-row strip
        upp = (p->shape == 2 && d->quadRows == 4) ? 4u : 1u;
        const uint32_t num_units = d->P * upp;
        const uint32_t resident = uint32_t(c.num_cus) * 4u * 8u;   // 4 SIMDs x 8 wavefronts per CU
        slots = t.slots ? t.slots : resident;
        std::vector<uint32_t> quads;
        if (t.slots) {
            int64_t n = cute_partition(num_units, unit.data(), num_slabs, slots, nullptr, 0);
            if (n < 0) { delete p; return int(n); }
            quads.resize(uint64_t(n) * 4);
            cute_partition(num_units, unit.data(), num_slabs, slots, quads.data(), uint64_t(n));
        } else {
            uint64_t work = 0;
            uint64_t busy = 0;
            for (uint32_t q = 0; q < num_units; ++q)
                if (!to_rows[q / upp] && unit[q + 1] != unit[q]) { work += unit[q + 1] - unit[q]; ++busy; }
            const uint64_t mean = busy ? (work + busy - 1) / busy : 1;
            const uint64_t share = (work * num_slabs + resident - 1) / resident;
            // the mean only counts while it is short: a matrix whose few MFMA panels are all very long
            // (a handful of dense rows) must still be cut, or one wavefront walks a whole panel alone
            const uint32_t target = uint32_t(std::max<uint64_t>(std::max<uint64_t>(share, std::min<uint64_t>(mean, 16)), 8));
            // A launch that keeps every wavefront slot busy runs at the rate the memory system gathers B rows, and a
            // work item then advances about five times slower than one that runs alone (measured on the R-MAT
            // benchmark matrix: 0.39 us per list group alone, 1.7 us per group and slot under load).  So an item up to
            // six shares long still ends with the launch, and cutting it finer only adds partial tiles: such a launch
            // cuts at six shares, into pieces of four.  A launch that does not fill the device is bound by its longest
            // item instead and keeps the finer cut (twice the target, pieces of one target).
            const uint32_t limit = uint32_t(std::max<uint64_t>(2u * uint64_t(target), 6u * share));
            const uint32_t piece = limit > 2u * target ? uint32_t(4u * share) : target;
            for (uint32_t q = 0; q < num_units; ++q) {
                const uint32_t s = unit[q], e = unit[q + 1];
                if (s == e || to_rows[q / upp]) continue;
                const uint32_t nblk = e - s;
                if (nblk <= limit) {
                    quads.insert(quads.end(), {s, e, q, 0u});
                    continue;
                }
                const uint32_t pieces = (nblk + piece - 1) / piece;
                const uint32_t step = (nblk + pieces - 1) / pieces;
                for (uint32_t cs = s; cs < e; cs += step) quads.insert(quads.end(), {cs, std::min(e, cs + step), q, 1u});
            }
        }
        // A chunk of a cut panel carries the 1-based number of its partial tile; the pieces of one panel are
        // consecutive (panels ascend through the list), and one fixup entry per cut panel adds them up afterwards.
        chunks.clear();
        fixups.clear();
        n_pieces = 0;
        for (size_t i = 0; i + 3 < quads.size(); i += 4) {
            const uint32_t s = quads[i], e = quads[i + 1], pan = quads[i + 2];
            uint32_t cut = quads[i + 3];
            if (to_rows[pan / upp]) continue;
            const uint32_t len = e - s;
            const uint32_t cap = t.max_chunk_blocks ? t.max_chunk_blocks : len;
            if (len > cap) cut = 1;                    // cut further than the partition asked for
            const uint32_t step = std::min(cap, len);
            for (uint32_t cs = s; cs < e; cs += step) {
                if (cut) {
                    if (fixups.empty() || fixups.back().x != pan) fixups.push_back(make_uint4(pan, n_pieces, 0u, 0u));
                    fixups.back().z++;
                    ++n_pieces;
                }
                chunks.push_back(make_uint4(cs, std::min(e, cs + step), pan, cut ? n_pieces : 0u));
            }
        }
        // a strip without pairs inside an MFMA-routed panel still has to be written (as zeros): an empty chunk
        if (upp > 1)
            for (uint32_t q = 0; q < num_units; ++q)
                if (unit[q] == unit[q + 1] && !to_rows[q / upp]) chunks.push_back(make_uint4(unit[q], unit[q], q, 0u));
        const bool lean = p->shape == 2 || p->pipeline == 1;
        if (!lean || !n_pieces || cute_offsets_fit(d->M, d->K, N, 0, uint64_t(n_pieces) * (CUTE_TM / upp)) == 1) break;
        if (attempt || t.mfma_shape == 2 || t.pipeline == 1) { delete p; return CUTE_ERR_SHAPE; }   // the caller forced a fast kernel
        p->shape = 1;
        p->pipeline = 2;
        p->bf16x3 = false;
    }
    std::vector<uint32_t> row_list;
    for (uint32_t q = 0; q < d->P; ++q)
        if (to_rows[q])
            for (uint32_t r = 0; r < CUTE_TM; ++r) row_list.push_back(q * CUTE_TM + r);

    // Row-kernel blocks per XCD: contiguous ranges of rows (neighbouring rows share B rows, which then stay
    // in one L2), cut where the running work -- nonzeros plus a fixed cost per row -- passes each eighth.
    {
        const uint32_t items_per_block = 256u >> p->rows_logl;             // rows of one 256-thread block (per slab)
        const uint64_t total_items = uint64_t(row_list.size());
        const uint32_t total_blocks = uint32_t((total_items + items_per_block - 1) / items_per_block);
        uint64_t total_work = 0;
        for (uint32_t q = 0; q < d->P; ++q)
            if (to_rows[q]) total_work += d->panelNnz[q] + 4u * CUTE_TM;
        uint64_t work = 0, items = 0;
        uint32_t x = 1;
        p->rowRanges.first[0] = 0;
        for (uint32_t q = 0; q < d->P && x < cute_dev::kNumXcd; ++q) {
            if (!to_rows[q]) continue;
            work += d->panelNnz[q] + 4u * CUTE_TM;
            items += uint64_t(CUTE_TM);
            while (x < cute_dev::kNumXcd && work * cute_dev::kNumXcd >= total_work * x)
                p->rowRanges.first[x++] = uint32_t(std::min<uint64_t>(total_blocks, (items + items_per_block - 1) / items_per_block));
        }
        while (x <= cute_dev::kNumXcd) p->rowRanges.first[x++] = total_blocks;
        p->rowBlocksPerXcd = 0;
        for (uint32_t k = 0; k < cute_dev::kNumXcd; ++k)
            p->rowBlocksPerXcd = std::max(p->rowBlocksPerXcd, p->rowRanges.first[k + 1] - p->rowRanges.first[k]);
    }
    if (t.chunk_order > 3) { delete p; return CUTE_ERR_ARG; }
    p->info.dealtChunks = 0;
    // A launch larger than the device starts its work-groups in list order as slots come free, and every XCD walks
    // its own eighth of the list.  In panel order that goes wrong in two ways: long items that start late keep the
    // launch waiting, and a matrix whose heavy panels sit together (the hub vertices of an R-MAT graph are its first
    // rows) gives one XCD most of the work.  So if the items differ widely in length (the longest at least four times
    // the mean), or the eighths of the list differ by more than a tenth in work, the long items go first and the list
    // is dealt round-robin to the XCDs: items are ordered by the power of two of their length only, so neighbours of
    // similar length stay neighbours and keep sharing B rows in the L2.
    // Hub plans: the strips of a graph with hub vertices through persistent work-groups that keep the most
    // referenced B rows in LDS.  Opt-in (cute_tunables.hub_rows); needs the quad kernel on strip lists.
    const uint32_t hub_rows = (t.hub_rows && p->shape == 2 && d->quadRows == 4 && !chunks.empty())
                                  ? std::min<uint32_t>(std::min<uint32_t>(t.hub_rows, kMaxHubRows), d->K) : 0u;
    if (hub_rows) {
        // work items are dealt to the wavefronts of the resident work-groups in list order: longest first
        std::stable_sort(chunks.begin(), chunks.end(), [](const uint4 &a, const uint4 &b) { return a.y - a.x > b.y - b.x; });
        p->info.dealtChunks = 2;
    }
    bool longest_first = t.chunk_order == 3 && !hub_rows;
    if (t.chunk_order == 0 && !chunks.empty() && !hub_rows) {
        const uint64_t resident = uint64_t(c.num_cus) * 4u * ((p->shape == 2 || p->ng == 1) ? 8u : 4u);
        uint64_t total = 0;
        uint32_t longest = 0;
        for (const uint4 &ck : chunks) { total += ck.y - ck.x; longest = std::max(longest, ck.y - ck.x); }
        const uint32_t groups = (uint32_t(chunks.size()) + cute_dev::kWavesPerGroup - 1) / cute_dev::kWavesPerGroup;
        const size_t span = size_t((groups + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd) * cute_dev::kWavesPerGroup;
        uint64_t fullest = 0;
        for (uint32_t x = 0; x < cute_dev::kNumXcd; ++x) {
            uint64_t work = 0;
            for (size_t i = std::min(chunks.size(), x * span); i < std::min(chunks.size(), (x + 1) * span); ++i) work += chunks[i].y - chunks[i].x + 2u;
            fullest = std::max(fullest, work);
        }
        const uint64_t even = (total + 2u * chunks.size() + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd;
        longest_first = uint64_t(chunks.size()) * num_slabs > resident &&
                        (uint64_t(longest) * chunks.size() >= 4u * total || fullest * 10u > even * 11u);
    }
    if (longest_first && !chunks.empty()) {
        std::vector<uint4> sorted(chunks);
        std::stable_sort(sorted.begin(), sorted.end(), [](const uint4 &a, const uint4 &b) {
            return __builtin_clz((a.y - a.x) | 1u) < __builtin_clz((b.y - b.x) | 1u);
        });
        // work-group g runs on XCD g % 8 and takes the list positions the kernels' XCD mapping gives it: XCD x walks
        // the groups [x * per_xcd, (x + 1) * per_xcd).  Deal the sorted groups round-robin into those ranges.
        const uint32_t wpg = cute_dev::kWavesPerGroup;
        const uint32_t groups = (uint32_t(sorted.size()) + wpg - 1) / wpg;
        const uint32_t per_xcd = (groups + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd;
        uint32_t fill[cute_dev::kNumXcd] = {}, cap[cute_dev::kNumXcd];
        for (uint32_t x = 0; x < cute_dev::kNumXcd; ++x)
            cap[x] = uint32_t(std::min<uint64_t>(per_xcd, groups > x * per_xcd ? groups - x * per_xcd : 0));
        // the last group may be short: it must stay the last one of the list
        const bool ragged = sorted.size() % wpg != 0;
        uint32_t last_xcd = 0;
        for (uint32_t x = 0; x < cute_dev::kNumXcd; ++x) if (cap[x]) last_xcd = x;
        if (ragged) cap[last_xcd]--;
        for (uint32_t k = 0; k < groups - (ragged ? 1u : 0u); ++k) {
            uint32_t x = k % cute_dev::kNumXcd;
            while (fill[x] == cap[x]) x = (x + 1) % cute_dev::kNumXcd;
            const size_t dst = (size_t(x) * per_xcd + fill[x]++) * wpg;
            for (uint32_t w = 0; w < wpg; ++w) chunks[dst + w] = sorted[size_t(k) * wpg + w];
        }
        if (ragged) {
            const size_t dst = (size_t(last_xcd) * per_xcd + cap[last_xcd]) * wpg, src = size_t(groups - 1) * wpg;
            for (size_t w = 0; src + w < sorted.size(); ++w) chunks[dst + w] = sorted[src + w];
        }
        p->info.dealtChunks = 2;
    } else
    if (t.chunk_order != 1 && !hub_rows && c.whole_chip && (p->shape == 2 || p->pipeline == 1) && !chunks.empty())
        p->info.dealtChunks = deal_chunks(chunks, num_slabs, uint32_t(c.num_cus) / cute_dev::kNumXcd,
                                          p->shape == 2 || p->ng == 1 ? 8u : 4u, t.chunk_order == 2) ? 1u : 0u;
    // the layout this plan's MFMA kernel reads, if the upload has not built it
    int rc = chunks.empty() ? int(CUTE_OK) : ensure_layout(d, p->shape);
    if (rc == CUTE_OK) rc = upload(&p->dChunks, chunks.data(), chunks.size());
    if (rc == CUTE_OK && hub_rows) rc = make_hub_tables(p, d, hub_rows);
    if (rc == CUTE_OK && p->shape == 2 && !chunks.empty()) {
        // one 128-byte head per work item: its descriptor and a copy of its first group's record, so that a
        // wavefront can ask for its first B rows after one scalar fetch instead of two dependent ones; gathered
        // on the device, where the records are
        const uint64_t words = uint64_t(chunks.size()) * cute_dev::kQuadHeadWords;
        if (hipMalloc(reinterpret_cast<void **>(&p->dHeads), words * sizeof(uint32_t)) != hipSuccess) rc = CUTE_ERR_NOMEM;
        if (rc == CUTE_OK) {
            hipLaunchKernelGGL(cute_build::quad_heads, grid_of(words), dim3(cute_build::kThreads), 0, nullptr, p->dChunks,
                               uint32_t(chunks.size()), p->dHubRecs ? p->dHubRecs : d->dQRecs, uint32_t(cute_dev::kQuadHeadWords), p->dHeads);
            rc = check_launch("quad heads");
            if (rc == CUTE_OK && hipStreamSynchronize(nullptr) != hipSuccess) rc = CUTE_ERR_HIP;
        }
    }
    if (rc == CUTE_OK) rc = upload(&p->dFixups, fixups.data(), fixups.size());
    p->unitRows = CUTE_TM / upp;
    // reduce_partials walks a tile along grid.y, a block of sixteen wavefronts taking 16 / G segments of 64 elements, G = 1..16
    // wavefronts to a segment by the number of pieces (see the kernel): the launch gets the blocks its tile with the most
    // pieces needs (the others leave theirs early), not one per segment -- with thousands of cut panels of two or three
    // pieces each the blocks that only start and exit otherwise cost more than the sums
    if (rc == CUTE_OK && n_pieces && (uint64_t(CUTE_TM / upp) * N + 63u) / 64u > 65535u) rc = CUTE_ERR_SHAPE;
    {
        uint32_t most = 1;
        for (const uint4 &fx : fixups) most = std::max(most, fx.z);
        const uint32_t G = most <= 4 ? 1u : most <= 8 ? 2u : most <= 16 ? 4u : most <= 32 ? 8u : 16u;    // as in reduce_partials
        const uint32_t segments = (CUTE_TM / upp * N + 63u) / 64u, per_block = uint32_t(cute_dev::kReduceWaves) / G;
        p->reduceBlocksY = std::max(1u, (segments + per_block - 1u) / per_block);
    }
    if (rc == CUTE_OK && n_pieces) {
        // (the fast kernels address the partial tiles like C, with 32-bit byte offsets: checked where the chunks were made)
        const uint64_t bytes = uint64_t(n_pieces) * p->unitRows * N * sizeof(float);
        p->partialBytes = bytes;
        if (hipMalloc(reinterpret_cast<void **>(&p->dPartials), bytes) != hipSuccess) rc = CUTE_ERR_NOMEM;
    }
    if (rc == CUTE_OK && !row_list.empty()) {
        // the list goes up as row indices and is packed with the rows' pointers on the device, where those are
        uint32_t *rows_only = nullptr;
        rc = upload(&rows_only, row_list.data(), row_list.size());
        if (rc == CUTE_OK && hipMalloc(reinterpret_cast<void **>(&p->dRowList), row_list.size() * sizeof(uint4)) != hipSuccess) rc = CUTE_ERR_NOMEM;
        if (rc == CUTE_OK) {
            hipLaunchKernelGGL(cute_build::pack_row_list, grid_of(row_list.size()), dim3(cute_build::kThreads), 0, nullptr, rows_only,
                               uint32_t(row_list.size()), d->dRowPtr, p->dRowList);
            rc = check_launch("row list");
            if (rc == CUTE_OK && hipStreamSynchronize(nullptr) != hipSuccess) rc = CUTE_ERR_HIP;
        }
        (void)hipFree(rows_only);
    }
    if (rc == CUTE_OK) {
        // cute_spmm_run_static's scratch: its address on this device is looked up here, at set-up, so that the
        // run call itself is nothing but kernel launches
        rc = static_scratch(&p->staticScratch);
    }
    if (rc != CUTE_OK) { cute_spmm_plan_free(p); return rc; }
    p->numFixups = uint32_t(fixups.size());
    p->numRows = uint32_t(row_list.size());
    p->info.N = N;
    p->info.slabWidth = slab;
    p->info.numSlabs = num_slabs;
    p->info.numChunks = uint32_t(chunks.size());
    p->info.numAtomicChunks = n_pieces;      // chunks of cut panels (the field keeps its name from the atomics they once used)
    p->info.numBrickPanels = n_brick;
    p->info.numRowPanelsSparse = n_rows;
    p->info.numEmptyPanels = n_empty;
    p->info.slots = slots;
    p->info.precision = p->bf16x3 ? uint32_t(CUTE_PREC_BF16X3) : uint32_t(CUTE_PREC_FP32);
    p->info.path = uint32_t(t.path);
    p->info.mfmaShape = uint32_t(p->shape);
    p->info.hubRows = p->numHub;
    p->info.pipeline = uint32_t(p->pipeline);
    // one launch for a mixed plan: the quad kernel with any row shape of 4-float lanes, the rolling brick
    // kernel in the shapes the planner itself picks for N (forced column groups fall back to two launches)
    const bool rows_fusable = !chunks.empty() && !row_list.empty() && p->rows_vec == 4;
    const bool brick_default_shape = ng_for_mixed || p->ng == ((p->vec == 4 && N >= 128) ? 2 : 1);
    p->info.partialTileKiB = uint32_t((p->partialBytes + 1023u) / 1024u);
    p->info.fusedLaunch = (rows_fusable && !p->bf16x3 && !p->numHub && (p->shape == 2 || (p->pipeline == 1 && brick_default_shape))) ? 1u : 0u;
    *out = p;
    return CUTE_OK;
}

}  // extern "C"

namespace {

template <int VEC, int NG, bool FULL>
void launch_brick_full(const cute_spmm_plan *p, const float *dB, float *dC, float *partials, hipStream_t s)
{
    const uint32_t groups = (p->info.numChunks + cute_dev::kWavesPerGroup - 1) / cute_dev::kWavesPerGroup;
    const uint32_t per_xcd = (groups + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd;
    const dim3 grid(per_xcd * cute_dev::kNumXcd, p->info.numSlabs), block(cute_dev::kWaveSize * cute_dev::kWavesPerGroup);
    if (p->bf16x3) {
        if constexpr (VEC == 4)
            hipLaunchKernelGGL((cute_dev::hrpb_brick_bf16x3<NG, FULL>), grid, block, 0, s, p->dChunks, p->info.numChunks, per_xcd,
                               p->d->dHdr, p->d->dVals, uint32_t(p->d->numVals), dB, dC, partials, p->info.N);
    } else if (p->pipeline == 1)
        hipLaunchKernelGGL((cute_dev::hrpb_brick_f32_rolling<VEC, NG, FULL>), grid, block, 0, s, p->dChunks,
                           p->info.numChunks, per_xcd, p->d->dHdr, p->d->dVals, uint32_t(p->d->numVals), dB, dC, partials, p->info.N);
    else
        hipLaunchKernelGGL((cute_dev::hrpb_brick_f32<VEC, NG, FULL>), grid, block, 0, s, p->dChunks, p->info.numChunks,
                           per_xcd, p->d->dHdr, p->d->dVals, dB, dC, partials, p->info.N);
}

template <int VEC, int NG>
void launch_brick(const cute_spmm_plan *p, const float *dB, float *dC, float *partials, hipStream_t s)
{
    if (p->info.N % p->info.slabWidth == 0) launch_brick_full<VEC, NG, true>(p, dB, dC, partials, s);
    else launch_brick_full<VEC, NG, false>(p, dB, dC, partials, s);
}

template <int VEC, bool BATCHED>
void launch_rows_vec(int logl, const uint4 *row_list, uint32_t num_rows, uint32_t slabs, const uint32_t *rp,
                     const uint32_t *cl, const float *vl, const float *dB, float *dC, uint32_t N, hipStream_t s,
                     const cute_dev::XcdRanges *ranges, uint32_t blocks_per_xcd)
{
    const uint64_t lanes = (uint64_t(num_rows) * slabs) << logl;
    // the batched kernel deals its blocks to the XCDs in contiguous ranges (all as long as the longest)
    const uint32_t blocks = uint32_t((lanes + 255) / 256);
    // the batched kernel walks the slabs in the grid's y dimension; the plain one folds them into x
    const dim3 grid(BATCHED ? blocks_per_xcd * cute_dev::kNumXcd : blocks, BATCHED ? slabs : 1u), block(256);
    const cute_dev::XcdRanges rg = ranges ? *ranges : cute_dev::XcdRanges{};
#define CUTE_ROWS_CASE(LL)                                                                                        \
    case LL:                                                                                                      \
        if (BATCHED)                                                                                              \
            hipLaunchKernelGGL((cute_dev::csr_rows_batched<VEC, LL, 8>), grid, block, 0, s, row_list, num_rows,    \
                               rp, cl, vl, dB, dC, N, rg);                                                        \
        else                                                                                                      \
            hipLaunchKernelGGL((cute_dev::csr_rows<VEC, LL>), grid, block, 0, s, static_cast<const uint32_t *>(nullptr), num_rows, slabs, rp, \
                               cl, vl, dB, dC, N);                                                                \
        break;
    switch (logl) {
        CUTE_ROWS_CASE(0) CUTE_ROWS_CASE(1) CUTE_ROWS_CASE(2) CUTE_ROWS_CASE(3)
        CUTE_ROWS_CASE(4) CUTE_ROWS_CASE(5) CUTE_ROWS_CASE(6)
    }
#undef CUTE_ROWS_CASE
}

// batched: the library's sparse-panel kernel; otherwise the plain comparison kernel
template <bool BATCHED>
void launch_rows(int vec, int logl, const uint4 *row_list, uint32_t num_rows, uint32_t slabs, const uint32_t *rp,
                 const uint32_t *cl, const float *vl, const float *dB, float *dC, uint32_t N, hipStream_t s,
                 const cute_dev::XcdRanges *ranges = nullptr, uint32_t blocks_per_xcd = 0)
{
    if (vec == 4) launch_rows_vec<4, BATCHED>(logl, row_list, num_rows, slabs, rp, cl, vl, dB, dC, N, s, ranges, blocks_per_xcd);
    else if (vec == 2) launch_rows_vec<2, BATCHED>(logl, row_list, num_rows, slabs, rp, cl, vl, dB, dC, N, s, ranges, blocks_per_xcd);
    else launch_rows_vec<1, BATCHED>(logl, row_list, num_rows, slabs, rp, cl, vl, dB, dC, N, s, ranges, blocks_per_xcd);
}

int check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, what, __LINE__);
    return CUTE_OK;
}

int csr_launch(int alg, const uint32_t *rp, const uint32_t *cl, const float *vl, const float *dB, float *dC, uint32_t M,
               uint32_t N, hipStream_t s)
{
    if (M == 0 || N == 0) return CUTE_ERR_SHAPE;
    switch (alg) {
        case 0:
            hipLaunchKernelGGL(cute_dev::csr_thread_per_element, dim3((N + 63) / 64, (M + 3) / 4), dim3(64, 4), 0, s, rp,
                               cl, vl, dB, dC, M, N);
            break;
        case 1:
            hipLaunchKernelGGL(cute_dev::csr_wave_scalar, dim3(uint32_t((uint64_t(M) * 64 + 255) / 256)), dim3(256), 0,
                               s, rp, cl, vl, dB, dC, M, N);
            break;
        case 2: {
            const int vec = (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
            uint32_t need = (N + vec - 1) / vec, logl = 0;
            while ((1u << logl) < need && logl < 6) ++logl;
            const uint32_t w = (1u << logl) * vec;
            launch_rows<false>(vec, int(logl), nullptr, M, (N + w - 1) / w, rp, cl, vl, dB, dC, N, s);
            break;
        }
        default: return CUTE_ERR_ARG;
    }
    return check_launch("csr kernel launch");
}

}  // namespace

namespace {
template <class Launch>
int time_launches(hipStream_t s, int warmup, int iters, float *ms_out, Launch launch)
{
    if (iters < 1 || !ms_out) return CUTE_ERR_ARG;
    std::vector<hipEvent_t> ev(size_t(iters) * 2, nullptr);
    int rc = CUTE_OK;
    for (auto &e : ev)
        if (rc == CUTE_OK && hipEventCreate(&e) != hipSuccess) rc = CUTE_ERR_HIP;
    for (int i = 0; i < warmup && rc == CUTE_OK; ++i) rc = launch();
    for (int i = 0; i < iters && rc == CUTE_OK; ++i) {
        (void)hipEventRecord(ev[2 * i], s);
        rc = launch();
        (void)hipEventRecord(ev[2 * i + 1], s);
    }
    if (rc == CUTE_OK && hipStreamSynchronize(s) != hipSuccess) rc = CUTE_ERR_HIP;
    for (int i = 0; i < iters && rc == CUTE_OK; ++i)
        if (hipEventElapsedTime(&ms_out[i], ev[2 * i], ev[2 * i + 1]) != hipSuccess) rc = CUTE_ERR_HIP;
    for (auto &e : ev)
        if (e) (void)hipEventDestroy(e);
    return rc;
}
}  // namespace

struct cute_blocked_ell_dev {
    int32_t blockSize = 0, height = 0, width = 0;
    int32_t *dColIdx = nullptr;
    float *dValues = nullptr;
};

struct cute_hybrid {
    cute_hybrid_info info{};
    uint32_t rows = 0;
    cute_blocked_ell_dev *ell = nullptr;    // heavy tiles (absent when no tile is heavy)
    uint32_t *dRowPtr = nullptr, *dCols = nullptr;
    float *dVals = nullptr;                 // the remainder as CSR
};

namespace {
template <int VEC, bool ACC>
void launch_blocked_ell(const cute_blocked_ell_dev *d, const float *dB, float *dC, uint32_t N, hipStream_t s)
{
    const uint32_t rows = uint32_t(d->height) * uint32_t(d->blockSize), strips = rows / 16u;
    // x extent a multiple of the XCD count: the kernel maps x so that each XCD owns a contiguous range of strips
    const uint32_t groups = (((strips + 3u) / 4u + 7u) / 8u) * 8u;
    const dim3 grid(groups, (N + 16u * VEC - 1u) / (16u * VEC)), block(256);
    if (N % (16u * VEC) == 0)
        hipLaunchKernelGGL((cute_dev::blocked_ell_f32<VEC, true, ACC>), grid, block, 0, s, d->dColIdx, d->dValues,
                           uint32_t(d->blockSize), uint32_t(d->width), strips, rows, dB, dC, N);
    else
        hipLaunchKernelGGL((cute_dev::blocked_ell_f32<VEC, false, ACC>), grid, block, 0, s, d->dColIdx, d->dValues,
                           uint32_t(d->blockSize), uint32_t(d->width), strips, rows, dB, dC, N);
}
}  // namespace

namespace {
// Brick chunks and sparse rows in one launch.  (VEC, NG, lanes per row) follow from N the way the planner
// picks them; returns false for a combination that is not instantiated (the caller then launches twice).
template <int VEC, int NG, int LOG_L>
void launch_brick_rows_as(const cute_spmm_plan *p, const float *dB, float *dC, float *partials, hipStream_t s, const dim3 &grid,
                          uint32_t per_xcd)
{
    const uint32_t N = p->info.N;
    const uint32_t rows_per_slab = p->rowBlocksPerXcd * cute_dev::kNumXcd;
    const uint64_t brick_blocks = uint64_t(grid.x) * grid.y, row_blocks = uint64_t(rows_per_slab) * p->rows_slabs;
    const dim3 flat(uint32_t(brick_blocks + row_blocks)), block(cute_dev::kWaveSize * cute_dev::kWavesPerGroup);
#define CUTE_BRICK_ROWS(F)                                                                                                \
    hipLaunchKernelGGL((cute_dev::hrpb_brick_rows_f32<VEC, NG, F, LOG_L>), flat, block, 0, s, grid.x, uint32_t(brick_blocks),  \
                       p->dChunks, p->info.numChunks, per_xcd, p->d->dHdr, p->d->dVals, uint32_t(p->d->numVals), p->dRowList, \
                       p->numRows, rows_per_slab, p->rowRanges, p->d->dRowPtr, p->d->dCols, p->d->dCsrVals,                    \
                       dB, dC, partials, N)
    if (N % (16u * VEC * NG) == 0) CUTE_BRICK_ROWS(true);
    else CUTE_BRICK_ROWS(false);
#undef CUTE_BRICK_ROWS
}

bool launch_brick_rows(const cute_spmm_plan *p, const float *dB, float *dC, float *partials, hipStream_t s)
{
    const uint32_t groups = (p->info.numChunks + cute_dev::kWavesPerGroup - 1) / cute_dev::kWavesPerGroup;
    const uint32_t per_xcd = (groups + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd;
    const dim3 grid(per_xcd * cute_dev::kNumXcd, p->info.numSlabs);
    if (uint64_t(grid.x) * grid.y + uint64_t(p->rowBlocksPerXcd) * cute_dev::kNumXcd * p->rows_slabs >= 0x7fffffffull) return false;
    const int v = p->vec, g = p->ng, l = p->rows_logl;
    if (v == 1 && g == 1 && l == 0) launch_brick_rows_as<1, 1, 0>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 1 && g == 1 && l == 1) launch_brick_rows_as<1, 1, 1>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 1 && g == 1 && l == 2) launch_brick_rows_as<1, 1, 2>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 2 && g == 1 && l == 3) launch_brick_rows_as<2, 1, 3>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 4 && g == 1 && l == 4) launch_brick_rows_as<4, 1, 4>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 4 && g == 1 && l == 5) launch_brick_rows_as<4, 1, 5>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 4 && g == 1 && l == 6) launch_brick_rows_as<4, 1, 6>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 4 && g == 2 && l == 5) launch_brick_rows_as<4, 2, 5>(p, dB, dC, partials, s, grid, per_xcd);
    else if (v == 4 && g == 2 && l == 6) launch_brick_rows_as<4, 2, 6>(p, dB, dC, partials, s, grid, per_xcd);
    else return false;
    return true;
}
}  // namespace

namespace {
// The launches of one product; `partials` is where the pieces of cut panels store their tiles.
int run_with(const cute_spmm_plan *p, const float *dB, float *dC, void *stream, float *partials)
{
    if (!p || !dB || !dC) return CUTE_ERR_ARG;
    if ((reinterpret_cast<uintptr_t>(dB) | reinterpret_cast<uintptr_t>(dC)) & 15u) return CUTE_ERR_ARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t N = p->info.N;
    bool rows_launched = false;        // the sparse rows went out together with the MFMA chunks
    if (p->info.numChunks && p->shape == 2 && p->numHub) {
        // persistent work-groups of sixteen wavefronts, two per compute unit, each with the hub rows of its slab in LDS
        const uint32_t wgs = std::min<uint32_t>(2u * uint32_t(context().num_cus), (p->info.numChunks + cute_dev::kHubWaves - 1) / cute_dev::kHubWaves);
        const dim3 grid(wgs, p->info.numSlabs), block(cute_dev::kWaveSize * cute_dev::kHubWaves);
        const size_t lds = size_t(p->numHub) * cute_dev::kWaveSize * sizeof(float);
        if (N % 64u == 0)
            hipLaunchKernelGGL((cute_dev::hrpb_quad_hub_f32<true>), grid, block, lds, s, p->dHeads, p->info.numChunks, p->dHubRecs,
                               p->d->dQVals, uint32_t(p->d->numQuadVals), p->dHubRows, p->numHub, dB, dC, partials, N);
        else
            hipLaunchKernelGGL((cute_dev::hrpb_quad_hub_f32<false>), grid, block, lds, s, p->dHeads, p->info.numChunks, p->dHubRecs,
                               p->d->dQVals, uint32_t(p->d->numQuadVals), p->dHubRows, p->numHub, dB, dC, partials, N);
    } else if (p->info.numChunks && p->shape == 2) {
        const uint32_t groups = (p->info.numChunks + cute_dev::kWavesPerGroup - 1) / cute_dev::kWavesPerGroup;
        const uint32_t per_xcd = (groups + cute_dev::kNumXcd - 1) / cute_dev::kNumXcd;
        const dim3 grid(per_xcd * cute_dev::kNumXcd, p->info.numSlabs), block(cute_dev::kWaveSize * cute_dev::kWavesPerGroup);
        const bool full = N % 64u == 0, strips = p->d->quadRows == 4;
        // mixed plan: quad chunks and sparse rows in one launch (instantiated for 4-float lanes and 4..64 lanes per row)
        const uint32_t rows_per_slab = p->rowBlocksPerXcd * cute_dev::kNumXcd;
        const uint64_t row_blocks = uint64_t(rows_per_slab) * p->rows_slabs, quad_blocks = uint64_t(grid.x) * grid.y;
        if (p->info.fusedLaunch && quad_blocks + row_blocks < 0x7fffffffull) {
#define CUTE_FUSED_LAUNCH(F, S, LL)                                                                                       \
    hipLaunchKernelGGL((cute_dev::hrpb_quad_rows_f32<F, S, LL>), dim3(uint32_t(quad_blocks + row_blocks)), block, 0, s,     \
                       grid.x, uint32_t(quad_blocks), p->dHeads, p->info.numChunks, per_xcd, p->d->dQRecs, p->d->dQVals,   \
                       uint32_t(p->d->numQuadVals),                                                                  \
                       p->dRowList, p->numRows, rows_per_slab, p->rowRanges, p->d->dRowPtr, p->d->dCols, p->d->dCsrVals, dB, dC,    \
                       partials, N)
#define CUTE_FUSED_LL(F, S)                                                     \
    switch (p->rows_logl) {                                                     \
        case 0: CUTE_FUSED_LAUNCH(F, S, 0); break;                              \
        case 1: CUTE_FUSED_LAUNCH(F, S, 1); break;                              \
        case 2: CUTE_FUSED_LAUNCH(F, S, 2); break;                              \
        case 3: CUTE_FUSED_LAUNCH(F, S, 3); break;                              \
        case 4: CUTE_FUSED_LAUNCH(F, S, 4); break;                              \
        case 5: CUTE_FUSED_LAUNCH(F, S, 5); break;                              \
        default: CUTE_FUSED_LAUNCH(F, S, 6); break;                             \
    }
            if (full && strips) { CUTE_FUSED_LL(true, true) }
            else if (full) { CUTE_FUSED_LL(true, false) }
            else if (strips) { CUTE_FUSED_LL(false, true) }
            else { CUTE_FUSED_LL(false, false) }
#undef CUTE_FUSED_LL
#undef CUTE_FUSED_LAUNCH
            rows_launched = true;
        } else {
#define CUTE_QUAD_LAUNCH(F, S)                                                                                          \
    hipLaunchKernelGGL((cute_dev::hrpb_quad_f32<F, S>), grid, block, 0, s, p->dHeads, p->info.numChunks, per_xcd,         \
                       p->d->dQRecs, p->d->dQVals, uint32_t(p->d->numQuadVals), dB, dC, partials, N)
        if (full && strips) CUTE_QUAD_LAUNCH(true, true);
        else if (full) CUTE_QUAD_LAUNCH(true, false);
        else if (strips) CUTE_QUAD_LAUNCH(false, true);
        else CUTE_QUAD_LAUNCH(false, false);
#undef CUTE_QUAD_LAUNCH
        }
    } else if (p->info.numChunks) {
        if (p->info.fusedLaunch && launch_brick_rows(p, dB, dC, partials, s)) rows_launched = true;
        else if (p->vec == 4 && p->ng == 2) launch_brick<4, 2>(p, dB, dC, partials, s);
        else if (p->vec == 4) launch_brick<4, 1>(p, dB, dC, partials, s);
        else if (p->vec == 2) launch_brick<2, 1>(p, dB, dC, partials, s);
        else launch_brick<1, 1>(p, dB, dC, partials, s);
    }
    if (p->numRows && !rows_launched) {
        // every row: no list needed, which takes one dependent load out of each row's chain
        launch_rows<true>(p->rows_vec, p->rows_logl, p->numRows == p->d->M ? nullptr : p->dRowList, p->numRows, p->rows_slabs, p->d->dRowPtr, p->d->dCols,
                    p->d->dCsrVals, dB, dC, N, s, &p->rowRanges, p->rowBlocksPerXcd);
    }
    // panels that were cut: add their partial tiles up, in chunk order (no atomics, so a product is
    // the same bit for bit every time it is computed)
    if (p->numFixups)
        hipLaunchKernelGGL(cute_dev::reduce_partials, dim3(p->numFixups, p->reduceBlocksY),
                           dim3(cute_dev::kWaveSize * cute_dev::kReduceWaves), 0, s, p->dFixups, p->numFixups, p->unitRows,
                           partials, dC, N);
    return check_launch("spmm launch");
}
}  // namespace

extern "C" {

// Replaces SPMM_TC::run (spmm.cu:823-839): picks the kernel instantiation from N and
// launches asynchronously on `stream`.
int cute_spmm_run(cute_spmm_plan *p, const float *dB, float *dC, void *stream)
{
    if (!p) return CUTE_ERR_ARG;
    return run_with(p, dB, dC, stream, p->dPartials);
}

// The same launches with the partial tiles in the library's static device array instead of the plan's
// buffer: no allocation, no copy, no memset, no synchronisation -- kernel launches only.
int cute_spmm_run_static(cute_spmm_plan *p, const float *dB, float *dC, void *stream)
{
    if (!p) return CUTE_ERR_ARG;
    if (p->partialBytes > uint64_t(CUTE_STATIC_SCRATCH_BYTES)) {
        g_hip_error = "plan needs " + std::to_string(p->partialBytes) + " bytes of partial tiles, the static scratch holds " +
                      std::to_string(uint64_t(CUTE_STATIC_SCRATCH_BYTES));
        return CUTE_ERR_SCRATCH;
    }
    return run_with(p, dB, dC, stream, static_cast<float *>(p->staticScratch));   // the address was fetched when the plan was made
}

uint64_t cute_spmm_plan_scratch_bytes(const cute_spmm_plan *p) { return p ? p->partialBytes : 0; }

// The same launches with the partial tiles in memory the caller brings: one plan can then run on several
// streams at once, each call with a buffer of its own.
int cute_spmm_run_scratch(cute_spmm_plan *p, const float *dB, float *dC, void *stream, void *scratch, uint64_t scratch_bytes)
{
    if (!p) return CUTE_ERR_ARG;
    if (p->partialBytes) {
        if (!scratch || (reinterpret_cast<uintptr_t>(scratch) & 15u)) return CUTE_ERR_ARG;
        if (scratch_bytes < p->partialBytes) {
            g_hip_error = "plan needs " + std::to_string(p->partialBytes) + " bytes of partial tiles, the caller's scratch holds " +
                          std::to_string(scratch_bytes);
            return CUTE_ERR_SCRATCH;
        }
    }
    return run_with(p, dB, dC, stream, static_cast<float *>(scratch));
}

int cute_csr_spmm_dev(int alg, const uint32_t *dRowPtr, const uint32_t *dCols, const float *dVals, const float *dB,
                      float *dC, uint32_t M, uint32_t N, void *stream)
{
    if (!dRowPtr || !dB || !dC) return CUTE_ERR_ARG;
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    return csr_launch(alg, dRowPtr, dCols, dVals, dB, dC, M, N, static_cast<hipStream_t>(stream));
}


void cute_blocked_ell_dev_free(cute_blocked_ell_dev *d)
{
    if (!d) return;
    (void)hipFree(d->dColIdx);
    (void)hipFree(d->dValues);
    delete d;
}

int cute_blocked_ell_upload(const cute_blocked_ell *e, cute_blocked_ell_dev **out)
{
    if (!e || !out || e->blockSize <= 0 || e->height < 0 || e->width < 0) return CUTE_ERR_ARG;
    *out = nullptr;
    if (e->blockSize % 16) return CUTE_ERR_SHAPE;        // the kernel walks 16 x 16 tiles
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    cute_blocked_ell_dev *d = new cute_blocked_ell_dev;
    d->blockSize = e->blockSize; d->height = e->height; d->width = e->width;
    const uint64_t cells = uint64_t(e->height) * uint64_t(e->width);
    int rc = upload(&d->dColIdx, e->ellColIdx, cells);
    if (rc == CUTE_OK) rc = upload(&d->dValues, e->ellValues, cells * uint64_t(e->blockSize) * uint64_t(e->blockSize));
    if (rc != CUTE_OK) { cute_blocked_ell_dev_free(d); return rc; }
    *out = d;
    return CUTE_OK;
}


// C[height*blockSize x N] (+)= ELL . B[ncols x N], device pointers, asynchronous on `stream`.
int cute_blocked_ell_spmm(const cute_blocked_ell_dev *d, const float *dB, float *dC, uint32_t N, int accumulate, void *stream)
{
    if (!d || !dB || !dC) return CUTE_ERR_ARG;
    if (N == 0) return CUTE_ERR_SHAPE;
    if ((reinterpret_cast<uintptr_t>(dB) | reinterpret_cast<uintptr_t>(dC)) & 15u) return CUTE_ERR_ARG;
    if (d->height == 0) return CUTE_OK;
    if ((N + 15u) / 16u > 65535u) return CUTE_ERR_ARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int vec = (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
    if (accumulate) {
        if (vec == 4) launch_blocked_ell<4, true>(d, dB, dC, N, s);
        else if (vec == 2) launch_blocked_ell<2, true>(d, dB, dC, N, s);
        else launch_blocked_ell<1, true>(d, dB, dC, N, s);
    } else {
        if (vec == 4) launch_blocked_ell<4, false>(d, dB, dC, N, s);
        else if (vec == 2) launch_blocked_ell<2, false>(d, dB, dC, N, s);
        else launch_blocked_ell<1, false>(d, dB, dC, N, s);
    }
    return check_launch("blocked-ELL launch");
}

// ------------------------------------------------------------------------------------------------
// The hybrid the reference's earlier prototypes model (inc/SPMM.cuh:2528-2933 GPU_Compute_Multi_Kernel*,
// the 2-D variant at :2898: tiles with more than THRESHOLD entries go to the tensor cores as dense tiles,
// the rest to a plain kernel; inc/splitter.hpp and inc/preprocess.hpp:172-193 are its two split rules):
// heavy tiles as a Blocked-ELL matrix through blocked_ell_f32 (fp32 MFMA), the remainder through the CSR
// row kernel, both into one C.
// ------------------------------------------------------------------------------------------------
void cute_hybrid_free(cute_hybrid *h)
{
    if (!h) return;
    cute_blocked_ell_dev_free(h->ell);
    (void)hipFree(h->dRowPtr);
    (void)hipFree(h->dCols);
    (void)hipFree(h->dVals);
    delete h;
}

int cute_hybrid_create(const cute_csr_i32 *csr, int32_t tile_size, int32_t nnz_threshold, int32_t mode, float deviation_threshold,
                       float underload_dominance, cute_hybrid **out)
{
    if (!csr || !out || !csr->rowPtr || (mode != CUTE_HYBRID_SPLITTER && mode != CUTE_HYBRID_CLASSIFIER)) return CUTE_ERR_ARG;
    *out = nullptr;
    if (tile_size <= 0 || tile_size % 16 || csr->nrows <= 0 || csr->nrows % tile_size || csr->ncols % tile_size) return CUTE_ERR_SHAPE;
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return c.status;
    cute_hybrid *h = new cute_hybrid;
    h->info.tileSize = tile_size;
    h->info.mode = mode;
    h->rows = uint32_t(csr->nrows);
    int rc = cute_block_stats(csr, tile_size, h->info.stats);
    cute_split sp{};
    if (rc == CUTE_OK) {
        if (mode == CUTE_HYBRID_SPLITTER) {
            // Threshold 0: the fill from which a tile pays for itself on the matrix cores, measured on gfx950 with this
            // library's two kernels (16 384^2 matrices, a sparse background plus 20 000 tiles of a given fill, N = 128):
            // tiles 10 % full lose 10 us by moving to the Blocked-ELL part (37.6 against 27.9 us), tiles 20 % full win 9 us
            // (36.2 against 45.6), tiles 30 % full 28 us -- the break-even is near 15 % of the tile's cells.  And a heavy
            // part that would hold less than 2 % of the entries is not worth its own launch (14 tiles of the FEM
            // benchmark matrix: +9 us): everything then stays with the row kernel.
            const bool automatic = nnz_threshold <= 0;
            if (automatic) nnz_threshold = std::max(1, int32_t(std::ceil(kHybridFill * float(tile_size) * float(tile_size))));
            rc = cute_splitter_split(csr, tile_size, nnz_threshold, &sp);
            if (rc == CUTE_OK && automatic && sp.numHeavyElems && int64_t(sp.numHeavyElems) * 50 < int64_t(csr->nnz)) {
                cute_split_release(&sp);
                nnz_threshold = tile_size * tile_size + 1;
                rc = cute_splitter_split(csr, tile_size, nnz_threshold, &sp);
            }
        } else {
            rc = cute_split_by_class(csr, tile_size, deviation_threshold, underload_dominance, &sp);
            nnz_threshold = 0;
        }
    }
    h->info.threshold = nnz_threshold;
    cute_csr_i32 heavy{}, light{};
    cute_blocked_ell ell{};
    if (rc == CUTE_OK) {
        h->info.totalTiles = sp.totalTiles;
        h->info.heavyTiles = sp.numHeavyTiles; h->info.heavyElems = sp.numHeavyElems;
        h->info.lightTiles = sp.numLightTiles; h->info.lightElems = sp.numLightElems;
        rc = cute_coo_to_csr(&sp.light, &light);
    }
    if (rc == CUTE_OK && sp.numHeavyElems) rc = cute_coo_to_csr(&sp.heavy, &heavy);
    if (rc == CUTE_OK && sp.numHeavyElems) rc = cute_blocked_ell_build(&heavy, tile_size, &ell);
    if (rc == CUTE_OK && sp.numHeavyElems) {
        h->info.ellHeight = ell.height;
        h->info.ellWidth = ell.width;
        rc = cute_blocked_ell_upload(&ell, &h->ell);
    }
    if (rc == CUTE_OK) rc = upload(&h->dRowPtr, reinterpret_cast<const uint32_t *>(light.rowPtr), uint64_t(csr->nrows) + 1);
    if (rc == CUTE_OK) rc = upload(&h->dCols, reinterpret_cast<const uint32_t *>(light.cols), uint64_t(light.nnz));
    if (rc == CUTE_OK) rc = upload(&h->dVals, light.values, uint64_t(light.nnz));
    cute_blocked_ell_release(&ell);
    cute_csr_i32_release(&heavy);
    cute_csr_i32_release(&light);
    cute_split_release(&sp);
    if (rc != CUTE_OK) { cute_hybrid_free(h); return rc; }
    *out = h;
    return CUTE_OK;
}

int cute_hybrid_get_info(const cute_hybrid *h, cute_hybrid_info *out)
{
    if (!h || !out) return CUTE_ERR_ARG;
    *out = h->info;
    return CUTE_OK;
}

// C[nrows x N] = A . B: the remainder through the row kernel (which writes every row of C), then the heavy tiles
// added on top by the Blocked-ELL kernel; both asynchronous on `stream`, in that order.
int cute_hybrid_spmm(const cute_hybrid *h, const float *dB, float *dC, uint32_t N, void *stream)
{
    if (!h || !dB || !dC) return CUTE_ERR_ARG;
    if (N == 0) return CUTE_ERR_SHAPE;
    if ((reinterpret_cast<uintptr_t>(dB) | reinterpret_cast<uintptr_t>(dC)) & 15u) return CUTE_ERR_ARG;
    int rc = csr_launch(2, h->dRowPtr, h->dCols, h->dVals, dB, dC, h->rows, N, static_cast<hipStream_t>(stream));
    if (rc == CUTE_OK && h->ell) rc = cute_blocked_ell_spmm(h->ell, dB, dC, N, 1, stream);
    return rc;
}

// Shape of GPU_CSR_cuSPARSE_NEW (spmm.cu:860-960): host arrays in, host C out, one warm-up
// launch then `iters` timed launches between two events; returns ms per launch.
float cute_gpu_csr_spmm(const uint32_t *rowPtr, const uint32_t *cols, const float *vals, uint32_t nnz, const float *hB,
                        float *hC, uint32_t m, uint32_t k, uint32_t n, int iters, int alg)
{
    if (!rowPtr || !hB || !hC || iters < 1) return float(CUTE_ERR_ARG);
    const DeviceContext &c = context();
    if (c.status != CUTE_OK) return float(c.status);
    uint32_t *dR = nullptr, *dCl = nullptr;
    float *dV = nullptr, *dB = nullptr, *dC = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    float ms = 0.0f;
    int rc = upload(&dR, rowPtr, uint64_t(m) + 1);
    if (rc == CUTE_OK) rc = upload(&dCl, cols, nnz);
    if (rc == CUTE_OK) rc = upload(&dV, vals, nnz);
    if (rc == CUTE_OK) rc = upload(&dB, hB, uint64_t(k) * n);
    if (rc == CUTE_OK && hipMalloc(reinterpret_cast<void **>(&dC), uint64_t(m) * n * sizeof(float)) != hipSuccess)
        rc = CUTE_ERR_HIP;
    if (rc == CUTE_OK) rc = csr_launch(alg, dR, dCl, dV, dB, dC, m, n, nullptr);
    if (rc == CUTE_OK && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) rc = CUTE_ERR_HIP;
    if (rc == CUTE_OK) {
        (void)hipEventRecord(e0, nullptr);
        for (int i = 0; i < iters && rc == CUTE_OK; ++i) rc = csr_launch(alg, dR, dCl, dV, dB, dC, m, n, nullptr);
        (void)hipEventRecord(e1, nullptr);
        if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = CUTE_ERR_HIP;
    }
    if (rc == CUTE_OK && hipMemcpy(hC, dC, uint64_t(m) * n * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
        rc = CUTE_ERR_HIP;
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(dR); (void)hipFree(dCl); (void)hipFree(dV); (void)hipFree(dB); (void)hipFree(dC);
    return rc == CUTE_OK ? ms / float(iters) : float(rc);
}

int cute_spmm_time(cute_spmm_plan *p, const float *dB, float *dC, void *stream, int warmup, int iters, float *ms_out)
{
    if (!p) return CUTE_ERR_ARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return time_launches(s, warmup, iters, ms_out, [&] { return cute_spmm_run(p, dB, dC, stream); });
}

int cute_csr_spmm_time(int alg, const cute_hrpb_dev *d, const float *dB, float *dC, uint32_t N, void *stream, int warmup,
                       int iters, float *ms_out)
{
    if (!d) return CUTE_ERR_ARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return time_launches(s, warmup, iters, ms_out,
                         [&] { return csr_launch(alg, d->dRowPtr, d->dCols, d->dCsrVals, dB, dC, d->M, N, s); });
}

}  // extern "C"
