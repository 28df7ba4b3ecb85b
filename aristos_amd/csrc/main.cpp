// Benchmark driver with the protocol of the reference's runOS() (csrc/main.cu:13-73): one packed
// allocation, host data preparation in fp32 followed by conversion to Element, one host-to-device
// copy, forwardHostBench<32, 32>, and the line "epRank: 0 took X ms".
//
//   kleos_main [kleos_config.json]
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "kleos.hpp"

namespace {

#define HIP_OK(e)                                                                                  \
    do {                                                                                           \
        hipError_t c_ = (e);                                                                       \
        if (c_ != hipSuccess) {                                                                    \
            std::fprintf(stderr, "<%s:%d> %s:\n    %s: %s\n", __FILE__, __LINE__, #e,              \
                         hipGetErrorName(c_), hipGetErrorString(c_));                              \
            std::exit(1);                                                                          \
        }                                                                                          \
    } while (0)

// Counter-based normal generator: SplitMix64 hash of the element index, Box-Muller transform.
struct Normal {
    uint64_t key;
    float mean, std;
    static uint64_t mix(uint64_t x) {
        x += 0x9E3779B97F4A7C15ull;
        x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
        x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
        return x ^ (x >> 31);
    }
    float operator()(uint64_t i) const {
        const double u1 = (double((mix(key + 2 * i) >> 11)) + 1.0) * (1.0 / 9007199254740992.0);
        const double u2 = double(mix(key + 2 * i + 1) >> 11) * (1.0 / 9007199254740992.0);
        return mean + std * float(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
    }
};

uint16_t to_bf16(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return uint16_t(u >> 16);
}

}  // namespace

int main(int argc, char** argv) {
    const char* path = argc > 1 ? argv[1] : "kleos_config.json";
    kleos::initialize(path);
    const int rank = kleos::getRank();
    const kleos_config_t c = kleos::config();
    // element counts exactly as main.cu:23-30
    const uint64_t dZ = c.in_elems, cZ = c.in_elems + c.out_elems;
    char* p = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&p), cZ * sizeof(float)));
    HIP_OK(hipMemset(p, 0, cZ * sizeof(float)));
    std::vector<float> host(dZ, 0.0f);
    {
        // main.cu:42-58: N(0, 5) activations, gate weights for the E real experts, expert weights;
        // biases stay zero
        Normal dist{Normal::mix(47ull * uint64_t(rank + 42)), 0.0f, 5.0f};
        uint64_t n = 0;
        auto fill = [&](uint64_t off, uint64_t count) {
#pragma omp parallel for schedule(static)
            for (int64_t i = 0; i < int64_t(count); ++i) host[off + i] = dist(n + uint64_t(i));
            n += count;
        };
        fill(c.off_x, uint64_t(c.S) * c.H);
        fill(c.off_gate_w, uint64_t(c.E) * c.H);
        for (uint32_t e = 0; e < c.E; ++e) {
            fill(c.off_w_up + uint64_t(e) * c.I * c.H, uint64_t(c.I) * c.H);
            fill(c.off_w_down + uint64_t(e) * c.H * c.I, uint64_t(c.H) * c.I);
        }
    }
    if (c.elem_bytes == 2) {
        std::vector<uint16_t> elems(dZ);
        for (uint64_t i = 0; i < dZ; ++i) elems[i] = to_bf16(host[i]);   // main.cu:59-62
        HIP_OK(hipMemcpy(p, elems.data(), dZ * 2, hipMemcpyHostToDevice));
    } else {
        HIP_OK(hipMemcpy(p, host.data(), dZ * 4, hipMemcpyHostToDevice));
    }
    float timed = 0;
    kleos::moe::forwardHostBench<32, 32>(p, p + dZ * c.elem_bytes, timed);   // main.cu:68
    std::printf("epRank: %u took %.2fms\n", unsigned(rank), timed);         // main.cu:69
    HIP_OK(hipPeekAtLastError());
    kleos::finalize();
    HIP_OK(hipFree(p));
    return 0;
}
