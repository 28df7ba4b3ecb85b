// Host-callable launchers of the layer's kernels.
#pragma once
#include <hip/hip_runtime.h>

#include "layer.hpp"

namespace kleos_amd {

// Number of uint32 scheduler words the persistent kernel needs for a layer with these sizes.
size_t sched_words(uint32_t E, uint32_t cap_rows);
// Index of the word a persistent kernel sets when one of its bounded waits expired.
uint32_t sched_error_word();

// Phase launchers (KLEOS_MODE_PHASED). dtype: 0 fp32, 2 bf16.
hipError_t launch_gate(const LayerParams& p, int dtype, int num_cus, hipStream_t s);
// Ranges the gate splits the hidden dimension into when it computes its logits as a tiled product
// (16-bit Elements, more than 64 experts); 0 when it does not. LayerParams::gate_partial then holds
// splits * S * PX floats.
uint32_t gate_splits_for(uint32_t S, uint32_t H, uint32_t E, uint32_t PX, int dtype, int num_cus);
hipError_t launch_slots(const LayerParams& p, hipStream_t s);
hipError_t launch_expert_gemm(const LayerParams& p, int dtype, int kind /*0 up, 1 down*/, int num_cus, hipStream_t s);
hipError_t launch_combine(const LayerParams& p, int dtype, hipStream_t s);

// The whole layer as one persistent launch (KLEOS_MODE_FUSED). The plan fixes the grid (every
// workgroup resident at once), the LDS size and the scheduler constants for a configuration.
struct FusedPlan {
    const void* kernel = nullptr;
    uint32_t nwg = 0;
    uint32_t threads = 0;
    size_t smem = 0;
    uint32_t mt_max = 0;   // row blocks per expert at full capacity
    uint32_t lag = 0;      // experts between an up-projection segment and its down-projection segment
    bool cooperative = false;   // launch through hipLaunchCooperativeKernel (residency verified per launch)
};
hipError_t plan_fused(const LayerParams& p, int dtype, int num_cus, FusedPlan* plan);
// fused_seq: number of fused launches already issued on this scheduler arena.
// schedule: a KLEOS_SCHEDULE_* value.
hipError_t launch_fused(const LayerParams& p, const FusedPlan& plan, uint32_t fused_seq, int schedule, hipStream_t s);

// Measurement probe, no part of the layer: one launch of a loop of bf16 matrix instructions on
// operands held in registers (no LDS, no memory traffic inside the loop), on every CU, eight
// wavefronts each. tile 32: 32x32x16 instructions, tile 16: 16x16x32. `data`: at least
// kMfmaProbeWords 32-bit words the operands are drawn from (their bit patterns decide what the
// multipliers toggle), `sink`: one float nobody reads. Returns the flop count of the launch in *flop.
constexpr size_t kMfmaProbeWords = size_t(1) << 22;
hipError_t launch_mfma_probe(int tile, uint32_t iterations, const uint32_t* data, float* sink, int num_cus, double* flop,
                             hipStream_t s);
// Fills `words` 32-bit words with pairs of bf16 values of random sign and mantissa and exponents close to 1
// (zero = true: with zeros).
hipError_t launch_mfma_probe_fill(uint32_t* data, size_t words, bool zero, hipStream_t s);

// Why a configuration cannot run, or nullptr when it can.
const char* unsupported_reason(uint32_t E, uint32_t k);

}  // namespace kleos_amd
