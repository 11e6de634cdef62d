// Shared by the C++ restatements of the reference's operator tests.
#ifndef LNG_TEST_SUPPORT_HPP
#define LNG_TEST_SUPPORT_HPP

#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "lng_compute.hpp"

namespace support {

inline int failures = 0;

inline void expect(bool ok, const std::string &what) {
    if (!ok) {
        ++failures;
        std::printf("FAILED %s\n", what.c_str());
    }
}

// The generator of the reference's tests (metal-compute/tests/attention_grouped.rs:25-36,
// q8_0_and_gpt_oss_glue.rs:28-38): xorshift values in [-1, 1).
inline std::vector<float> values(uint64_t seed, size_t n) {
    std::vector<float> out(n);
    uint64_t s = seed | 1;
    for (size_t i = 0; i < n; ++i) {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        out[i] = (float)(s >> 40) / (float)(1ull << 23) - 1.0f;
    }
    return out;
}

inline lng::Buffer upload(const lng::Gpu &gpu, const std::vector<float> &v) {
    lng::Buffer b = gpu.buffer((v.empty() ? 1 : v.size()) * 4);
    b.copy_from_f32(v);
    return b;
}

inline lng::Buffer upload_bytes(const lng::Gpu &gpu, const std::vector<uint8_t> &v) {
    lng::Buffer b = gpu.buffer(v.size() < 16 ? 16 : v.size());
    if (!v.empty()) b.write(0, v.data(), v.size());
    return b;
}

inline lng::Slice f32s(size_t buffer, size_t n) { return lng::Slice(buffer, 0, n * 4); }

} // namespace support

#endif // LNG_TEST_SUPPORT_HPP
