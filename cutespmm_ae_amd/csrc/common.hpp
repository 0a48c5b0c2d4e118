// Shared host-side helpers of libcutespmm: allocation, a thread pool-less parallel_for,
// and the lane-order <-> canonical bitmap permutation used by the device layout.
#pragma once
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cctype>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/cutespmm.h"

namespace cute {

template <class T>
inline T *alloc_array(uint64_t n)
{
    return static_cast<T *>(std::calloc(n ? n : 1, sizeof(T)));
}

inline unsigned host_threads()
{
    unsigned n = std::thread::hardware_concurrency();
    if (const char *e = std::getenv("CUTE_NUM_THREADS")) {
        int v = std::atoi(e);
        if (v > 0) n = static_cast<unsigned>(v);
    }
    return std::max(1u, std::min(n, 64u));
}

// Calls fn(begin, end, thread_index) on contiguous ranges of [0, n).
template <class F>
inline void parallel_ranges(uint64_t n, uint64_t min_per_thread, F fn)
{
    unsigned nt = host_threads();
    if (min_per_thread == 0) min_per_thread = 1;
    nt = static_cast<unsigned>(std::min<uint64_t>(nt, (n + min_per_thread - 1) / min_per_thread));
    if (nt <= 1) {
        fn(uint64_t(0), n, 0u);
        return;
    }
    std::vector<std::thread> th;
    th.reserve(nt);
    for (unsigned t = 0; t < nt; ++t) {
        uint64_t b = n * t / nt, e = n * (t + 1) / nt;
        th.emplace_back([=] { fn(b, e, t); });
    }
    for (auto &x : th) x.join();
}

// Canonical brick bitmap: bit row*4+k (data.cu:36-38).  Lane order: bit k*16+row, the
// position of A[row][k] among the 64 lanes of a 16x16x4 fp32 MFMA A operand.
inline uint64_t bitmap_to_lane_order(uint64_t canon)
{
    uint64_t out = 0;
    while (canon) {
        unsigned b = static_cast<unsigned>(__builtin_ctzll(canon));
        canon &= canon - 1;
        out |= 1ull << ((b & 3u) * 16u + (b >> 2));
    }
    return out;
}
inline uint64_t bitmap_to_canonical(uint64_t lane)
{
    uint64_t out = 0;
    while (lane) {
        unsigned b = static_cast<unsigned>(__builtin_ctzll(lane));
        lane &= lane - 1;
        out |= 1ull << ((b & 15u) * 4u + (b >> 4));
    }
    return out;
}

// The banner line of a MatrixMarket file, "%%MatrixMarket matrix <format> <field> <symmetry>" (case-insensitive).
// The reference's readers only search that line for the substring "symmetric" (IO.cu:16,
// inc/SparseCoo.hpp:113); the value-keeping readers of this library tokenise it.
struct MmBanner {
    bool present = false;      // the line starts with %%MatrixMarket
    bool valid = false;        // object, format, field and symmetry are all known words
    bool array = false;        // format: array (dense, column-major) instead of coordinate
    int field = 0;             // 0 real, 1 integer, 2 pattern, 3 complex
    int symmetry = 0;          // 0 general, 1 symmetric, 2 skew-symmetric, 3 hermitian
};

inline MmBanner parse_mm_banner(const char *b, const char *e)
{
    MmBanner r;
    std::vector<std::string> tok;
    const char *s = b;
    while (s < e) {
        while (s < e && (*s == ' ' || *s == '\t' || *s == '\r')) ++s;
        const char *w = s;
        while (s < e && *s != ' ' && *s != '\t' && *s != '\r') ++s;
        if (s > w) {
            std::string t(w, s);
            for (char &ch : t) ch = char(std::tolower(static_cast<unsigned char>(ch)));
            tok.push_back(t);
        }
    }
    if (tok.empty() || tok[0] != "%%matrixmarket") return r;
    r.present = true;
    if (tok.size() != 5 || tok[1] != "matrix") return r;
    if (tok[2] == "array") r.array = true;
    else if (tok[2] != "coordinate") return r;
    const char *fields[4] = {"real", "integer", "pattern", "complex"};
    const char *syms[4] = {"general", "symmetric", "skew-symmetric", "hermitian"};
    int f = -1, y = -1;
    for (int i = 0; i < 4; ++i) {
        if (tok[3] == fields[i]) f = i;
        if (tok[4] == syms[i]) y = i;
    }
    if (f < 0 || y < 0 || (r.array && f == 2)) return r;     // a dense file cannot be a pattern
    r.field = f;
    r.symmetry = y;
    r.valid = true;
    return r;
}

// splitmix64: the counter-based generator behind every synthetic input.
inline uint64_t splitmix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
inline uint64_t rng_at(uint64_t seed, uint64_t stream, uint64_t idx)
{
    return splitmix64(splitmix64(seed ^ (stream << 56)) + idx);
}
inline float u01(uint64_t h) { return static_cast<float>(h >> 40) * (1.0f / 16777216.0f); }

}  // namespace cute
