// TEST INFRASTRUCTURE ONLY. C wrapper around the reference's own std-only header
// include/brodiffusion/detail/torch_rng.h, compiled from where it lies in the mounted
// reference tree (see oracle/Makefile, target _ref). It exists so the restated
// generator in oracle.cpp can be compared with the real one at arbitrary seeds and
// lengths. The built library goes to oracle/_ref/ and is never committed.
#include "brodiffusion/detail/torch_rng.h"

#include <cstdint>
#include <cstring>

extern "C" __attribute__((visibility("default")))
int ref_torch_randn_f32(uint64_t seed, size_t n, float* out) {
    try {
        const std::vector<float> v = brodiffusion::detail::torch_randn_f32(seed, n);
        std::memcpy(out, v.data(), n * sizeof(float));
        return 0;
    } catch (...) {
        return -1;
    }
}
