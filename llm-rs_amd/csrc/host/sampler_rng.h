// The reference's generator (src/sampler/mod.rs:2-25): xorshift64 with shifts
// 13, 7, 17; seed 0 stands for 0xDEADBEEFCAFE; a float in [0,1) is the top 24
// bits over 2^24.  Each request owns one state, so what it draws does not depend
// on the batch it is in.
#pragma once
#include <cstdint>

namespace llmrs {

struct Xorshift64 {
    uint64_t state;
    explicit Xorshift64(uint64_t seed = 42) : state(seed == 0 ? 0xDEADBEEFCAFEull : seed) {}
    uint64_t next_u64() {
        uint64_t x = state;
        x ^= x << 13;
        x ^= x >> 7;
        x ^= x << 17;
        state = x;
        return x;
    }
    float next_f32() { return (float)(next_u64() >> 40) / (float)(1ull << 24); }
};

}  // namespace llmrs
