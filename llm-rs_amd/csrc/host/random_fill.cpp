// Host twin of the device's seeded normal fill (csrc/hip/utility.hip): the same
// function of (seed, index), so a tensor made here equals, bit for bit, the one
// the device makes.  The range is shared out over threads; each value depends
// on its index alone.
#include <algorithm>
#include <cstddef>
#include <thread>
#include <vector>

#include "../shared/normal_stream.h"

namespace {

// Compiled twice: with hardware fused multiply-add where the processor has it,
// and without (the library's fmaf, exact as well, only slower); chosen at load.
__attribute__((target_clones("fma", "default")))
void fill_range(void* out, int dtype, size_t lo, size_t hi, uint64_t seed, uint64_t first, float mean, float std) {
    if (dtype == 1) {
        uint16_t* o = (uint16_t*)out;
        for (size_t i = lo; i < hi; ++i) o[i] = llmrs::ns_bf16_bits(llmrs::normal_value(seed, first + i, mean, std));
    } else {
        float* o = (float*)out;
        for (size_t i = lo; i < hi; ++i) o[i] = llmrs::normal_value(seed, first + i, mean, std);
    }
}

}  // namespace

// dtype: 0 float32, 1 bfloat16 (as the kernels' codes).  threads <= 0: as many as the machine has, at most 16.
extern "C" int llmrs_fill_normal_host(void* out, int dtype, size_t n, uint64_t seed, uint64_t first, float mean, float std,
                                      int threads) {
    if (dtype != 0 && dtype != 1) return -1;
    if (n == 0) return 0;
    if (out == nullptr) return -1;
    size_t want = threads > 0 ? (size_t)threads : std::min<size_t>(std::max(1u, std::thread::hardware_concurrency()), 16);
    size_t workers = std::max<size_t>(1, std::min(want, n / 65536 + 1));
    if (workers == 1) {
        fill_range(out, dtype, 0, n, seed, first, mean, std);
        return 0;
    }
    std::vector<std::thread> pool;
    size_t per = (n + workers - 1) / workers;
    for (size_t w = 0; w < workers; ++w) {
        size_t lo = w * per, hi = std::min(n, lo + per);
        if (lo >= hi) break;
        pool.emplace_back(fill_range, out, dtype, lo, hi, seed, first, mean, std);
    }
    for (auto& t : pool) t.join();
    return 0;
}
