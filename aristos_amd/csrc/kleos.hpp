// C++ host interface with the reference's names, over the C ABI in include/kleos_amd.h.
//
//   kleos::initialize / finalize / getRank / setDevice   (reference csrc/include/kleos/bootstrap.cuh:533-588)
//   kleos::moe::forwardHost / forwardHostBench           (reference csrc/include/kleos/moe/moe.cuh:146-205)
//
// The reference bakes its configuration in at compile time; here initialize() names the
// kleos_config.json to read. Errors keep the reference's convention (csrc/include/kleos/debug.cuh:
// 19-43): print the message and terminate the process.
#pragma once
#include <cstdio>
#include <cstdlib>

#include "../../include/kleos_amd.h"

#define KLEOS_AMD_CHECK(call)                                                         \
    do {                                                                              \
        const int kleos_rc_ = (call);                                                 \
        if (kleos_rc_ != KLEOS_OK) {                                                  \
            std::fprintf(stderr, "<%s:%d> %s:\n    Error: %s\n", __FILE__, __LINE__,  \
                         #call, kleos_last_error());                                  \
            std::fflush(stderr);                                                      \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

namespace kleos {

inline void initialize(const char* config_json_path = "kleos_config.json") {
    KLEOS_AMD_CHECK(kleos_initialize(config_json_path));
}
inline void initialize(const kleos_config_t& cfg) { KLEOS_AMD_CHECK(kleos_initialize_cfg(&cfg)); }
inline void finalize() { KLEOS_AMD_CHECK(kleos_finalize()); }
inline void setDevice() { KLEOS_AMD_CHECK(kleos_set_device()); }
inline int getRank() {
    const int r = kleos_get_rank();
    if (r < 0) {
        std::fprintf(stderr, "Error: %s\n", kleos_last_error());
        std::exit(1);
    }
    return r;
}
inline kleos_config_t config() {
    kleos_config_t c;
    KLEOS_AMD_CHECK(kleos_get_config(&c));
    return c;
}

namespace moe {

inline void forwardHost(const void* iP, void* oP) { KLEOS_AMD_CHECK(kleos_moe_forward(iP, oP)); }

template <unsigned skip = 50, unsigned trials = 100>
inline void forwardHostBench(const void* iP, void* oP, float& duration) {
    KLEOS_AMD_CHECK(kleos_moe_forward_bench(iP, oP, skip, trials, &duration));
}

}  // namespace moe
}  // namespace kleos
