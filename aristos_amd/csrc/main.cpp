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

// fp32 -> tf32 held in 32 bits: 10 mantissa bits, round to nearest even, the lower 13 bits cleared.
float to_tf32(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    if ((u & 0x7f800000u) != 0x7f800000u) u += 0x0fffu + ((u >> 13) & 1u);
    u &= 0xffffe000u;
    std::memcpy(&v, &u, 4);
    return v;
}

// fp32 -> IEEE binary16 bits, round to nearest even; overflow to infinity, gradual underflow.
uint16_t to_f16(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    const uint16_t sign = uint16_t((u >> 16) & 0x8000u);
    const uint32_t mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) return uint16_t(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u : 0u));   // inf / nan
    if (mag >= 0x477ff000u) return uint16_t(sign | 0x7c00u);   // rounds to 65520 or more: infinity
    if (mag < 0x33000001u) return sign;                        // at most half the smallest subnormal: zero
    int32_t exp = int32_t(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u;              // 24 significant bits
    // binary16 keeps 11 significant bits of a normal number, fewer below 2^-14
    const int shift = exp >= -14 ? 13 : 13 + (-14 - exp);
    const uint32_t kept = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t r = kept + uint32_t(rest > half || (rest == half && (kept & 1u)));
    // normal: r carries the implicit bit at position 10, so adding the biased exponent minus one
    // lets a carry out of the mantissa bump the exponent; subnormal: r is the mantissa itself
    const uint32_t bits = exp >= -14 ? (uint32_t(exp + 15 - 1) << 10) + r : r;
    return uint16_t(sign | bits);
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
        const bool f16 = c.torch_dtype == KLEOS_DTYPE_FP16;
        for (uint64_t i = 0; i < dZ; ++i) elems[i] = f16 ? to_f16(host[i]) : to_bf16(host[i]);   // main.cu:59-62
        HIP_OK(hipMemcpy(p, elems.data(), dZ * 2, hipMemcpyHostToDevice));
    } else {
        if (c.torch_dtype == KLEOS_DTYPE_TF32)
            for (uint64_t i = 0; i < dZ; ++i) host[i] = to_tf32(host[i]);   // main.cu:59-62, Element = tfloat32_t
        HIP_OK(hipMemcpy(p, host.data(), dZ * 4, hipMemcpyHostToDevice));
    }
    float timed = 0;
    kleos::moe::forwardHostBench<32, 32>(p, p + dZ * c.elem_bytes, timed);   // main.cu:68
    std::printf("epRank: %u took %.2fms\n", unsigned(rank), timed);         // main.cu:69
    HIP_OK(hipPeekAtLastError());
    if (std::getenv("KLEOS_MAIN_CHECK")) {
        // not in the reference's driver: the activations as the device holds them, decoded from the
        // configured Element type, must still be the N(0, 5) sample that was drawn on the host
        const uint64_t n = uint64_t(c.S) * c.H;
        std::vector<char> raw(n * c.elem_bytes);
        HIP_OK(hipMemcpy(raw.data(), p + c.off_x * c.elem_bytes, raw.size(), hipMemcpyDeviceToHost));
        double sum = 0.0, sq = 0.0, err = 0.0;
        for (uint64_t i = 0; i < n; ++i) {
            float v;
            if (c.elem_bytes == 4) {
                std::memcpy(&v, &raw[i * 4], 4);
            } else {
                uint16_t h;
                std::memcpy(&h, &raw[i * 2], 2);
                if (c.torch_dtype == KLEOS_DTYPE_FP16) {
                    const int e = (h >> 10) & 31, m = h & 1023;
                    v = e == 0 ? std::ldexp(float(m), -24) : (e == 31 ? INFINITY : std::ldexp(float(m | 1024), e - 25));
                    if (h & 0x8000u) v = -v;
                } else {
                    const uint32_t u = uint32_t(h) << 16;
                    std::memcpy(&v, &u, 4);
                }
            }
            sum += v; sq += double(v) * v;
            err = std::fmax(err, std::fabs(double(v) - host[c.off_x + i]) / (std::fabs(host[c.off_x + i]) + 1e-3));
        }
        std::printf("device x: mean %.4f std %.4f max relative conversion error %.5f\n", sum / double(n),
                    std::sqrt(sq / double(n)), err);
    }
    kleos::finalize();
    HIP_OK(hipFree(p));
    return 0;
}
