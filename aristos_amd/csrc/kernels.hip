// The part of the kernels' host interface that does not depend on the Element type: scheduler
// sizing, the slot kernel, the launch of a planned persistent kernel, and the switch over the
// Element type in front of the launchers that kernels_f32.hip, kernels_bf16.hip and kernels_f16.hip
// instantiate (kernels_impl.hpp).
#include "kernels_impl.hpp"

namespace kleos_amd {

KLEOS_EXTERN_ELEMENT(float)
KLEOS_EXTERN_ELEMENT(tf32_t)
KLEOS_EXTERN_ELEMENT(bf16_t)
KLEOS_EXTERN_ELEMENT(f16_t)

namespace {
__global__ __launch_bounds__(kPhaseThreads) void slot_kernel(const LayerParams p) {
    extern __shared__ uint32_t slot_smem[];
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t tile = blockIdx.x * 4 + wave;
    slot_tile(p, tile, tile < p.n_gate_tiles, slot_smem + wave * p.E);
    // the coarse counts of the other epoch are free now: clear them for the next launch
    uint32_t* other = p.super_count + size_t((p.epoch & 1u) ^ 1u) * p.n_super * p.E;
    for (uint32_t i = blockIdx.x * kPhaseThreads + threadIdx.x; i < p.n_super * p.E; i += gridDim.x * kPhaseThreads)
        other[i] = 0u;
}
}  // namespace

const char* unsupported_reason(uint32_t E, uint32_t k) {
    if (E > kMaxExperts) return "num_experts > 512 is not supported by this build (LDS tables of the persistent kernel)";
    if (E > 16 * kMaxGateGroups && k > kWideGateMaxK)
        return "expert_top_k > 32 with num_experts > 256 is not supported by the gate kernel of this build";
    return nullptr;
}

uint32_t sched_error_word() { return kSchedError; }


size_t sched_words(uint32_t E, uint32_t cap_rows) {
    return kSchedReady + size_t(E) * ceil_div_u32(cap_rows, 64) + 64;
}

uint32_t gate_splits_for(uint32_t S, uint32_t H, uint32_t E, uint32_t PX, int dtype, int num_cus) {
    if ((dtype != 2 && dtype != 3) || E <= 64) return 0;
    const uint32_t tiles = (S / kGateTileM) * ceil_div_u32(PX, kGateTileN);
    uint32_t splits = ceil_div_u32(uint32_t(num_cus), tiles ? tiles : 1u);
    const uint32_t slices = H / 64;
    if (splits > slices) splits = slices;
    if (splits > kGateMaxSplits) splits = kGateMaxSplits;
    return splits < 1 ? 1u : splits;
}

// Calls go(Element{}) for the Element type of a torch_dtype value (kleos_amd.h: 0 fp32, 1 tf32, 2 bf16, 3 fp16).
template <typename F>
hipError_t dispatch_dtype(int dtype, F&& go) {
    switch (dtype) {
        case 1: return go(tf32_t{});
        case 2: return go(bf16_t{});
        case 3: return go(f16_t{});
        default: return go(float{});
    }
}

hipError_t launch_gate(const LayerParams& p, int dtype, int num_cus, hipStream_t s) {
    return dispatch_dtype(dtype, [&](auto tag) { return launch_gate_t<decltype(tag)>(p, num_cus, s); });
}

hipError_t launch_slots(const LayerParams& p, hipStream_t s) {
    const uint32_t grid = ceil_div_u32(p.n_gate_tiles, 4);
    hipLaunchKernelGGL(slot_kernel, dim3(grid), dim3(kPhaseThreads), 4 * p.E * sizeof(uint32_t), s, p);
    return hipGetLastError();
}

hipError_t launch_expert_gemm(const LayerParams& p, int dtype, int kind, int num_cus, hipStream_t s) {
    return dispatch_dtype(dtype, [&](auto tag) { return launch_expert_gemm_t<decltype(tag)>(p, kind, num_cus, s); });
}

hipError_t launch_combine(const LayerParams& p, int dtype, hipStream_t s) {
    return dispatch_dtype(dtype, [&](auto tag) { return launch_combine_t<decltype(tag)>(p, s); });
}

hipError_t plan_fused(const LayerParams& p, int dtype, int num_cus, FusedPlan* plan) {
    return dispatch_dtype(dtype, [&](auto tag) { return plan_fused_t<decltype(tag)>(p, num_cus, plan); });
}

hipError_t launch_fused(const LayerParams& p, const FusedPlan& plan, uint32_t fused_seq, int schedule, hipStream_t s) {
    uint32_t seq = fused_seq;
    uint32_t mt_max = plan.mt_max, lag = plan.lag, policy = uint32_t(schedule);
    LayerParams pc = p;
    void* args[] = {&pc, &seq, &mt_max, &lag, &policy};
    // A cooperative launch makes the runtime verify that the whole grid can be resident at once
    // (it fails with hipErrorCooperativeLaunchTooLarge otherwise); it costs about 14 us per launch.
    if (plan.cooperative) return hipLaunchCooperativeKernel(plan.kernel, dim3(plan.nwg), dim3(plan.threads), args, plan.smem, s);
    return hipLaunchKernel(plan.kernel, dim3(plan.nwg), dim3(plan.threads), args, plan.smem, s);
}


// ------------------------------------------------------------------------------------ probe
namespace {
template <int TILE>
__global__ __launch_bounds__(512, 1) void mfma_probe_kernel(const uint32_t* data, float* sink, uint32_t iterations) {
    // eight operand fragments of each kind per lane, as a 128 x 64 wavefront tile keeps them around
    bf16x8 fa[8], fb[8];
    const u32x4* pool = reinterpret_cast<const u32x4*>(data);
    constexpr uint32_t kMask = uint32_t(kMfmaProbeWords / 4 - 1);
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
        fa[i] = __builtin_bit_cast(bf16x8, pool[(blockIdx.x * 512u + threadIdx.x + i * 4096u) & kMask]);
        fb[i] = __builtin_bit_cast(bf16x8, pool[(blockIdx.x * 512u + threadIdx.x + i * 4096u + 77777u) & kMask]);
    }
    float total = 0.f;
    if constexpr (TILE == 32) {
        f32x16 acc[2][4] = {};
        for (uint32_t it = 0; it < iterations; ++it)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int n = 0; n < 2; ++n)
#pragma unroll
                    for (int m = 0; m < 4; ++m)
                        acc[n][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[(n + 2 * ks) & 7], fa[(m + ks) & 7], acc[n][m], 0, 0, 0);
        for (int n = 0; n < 2; ++n) for (int m = 0; m < 4; ++m) for (int i = 0; i < 16; ++i) total += acc[n][m][i];
    } else {
        f32x4 acc[4][8] = {};
        for (uint32_t it = 0; it < iterations; ++it)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int n = 0; n < 4; ++n)
#pragma unroll
                    for (int m = 0; m < 8; ++m)
                        acc[n][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[(n + 4 * ks) & 7], fa[(m + ks) & 7], acc[n][m], 0, 0, 0);
        for (int n = 0; n < 4; ++n) for (int m = 0; m < 8; ++m) for (int i = 0; i < 4; ++i) total += acc[n][m][i];
    }
    if (total == 12345.678f) *sink = total;   // keeps the loop alive; never true in practice
}

__global__ void mfma_probe_fill_kernel(uint32_t* data, size_t words, uint32_t zero) {
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < words; i += size_t(gridDim.x) * blockDim.x) {
        uint32_t h = uint32_t(i) * 2654435761u + 12345u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13; h *= 3266489917u; h ^= h >> 16;
        // two bf16: sign and 7 mantissa bits random, exponent 0x7e or 0x7f (0.5 <= |v| < 2)
        const uint32_t lo = (h & 0x80ffu) | 0x3f00u, hi = ((h >> 16) & 0x80ffu) | 0x3f00u;
        data[i] = zero ? 0u : (lo | (hi << 16));
    }
}
}  // namespace

hipError_t launch_mfma_probe(int tile, uint32_t iterations, const uint32_t* data, float* sink, int num_cus, double* flop,
                             hipStream_t s) {
    if (tile != 16 && tile != 32) return hipErrorInvalidValue;
    // per iteration and wavefront: a 128 x 64 tile advanced by 64 values of K
    if (flop) *flop = double(num_cus) * 8.0 * double(iterations) * 2.0 * 128.0 * 64.0 * 64.0;
    if (tile == 32) hipLaunchKernelGGL(mfma_probe_kernel<32>, dim3(num_cus), dim3(512), 0, s, data, sink, iterations);
    else hipLaunchKernelGGL(mfma_probe_kernel<16>, dim3(num_cus), dim3(512), 0, s, data, sink, iterations);
    return hipGetLastError();
}

hipError_t launch_mfma_probe_fill(uint32_t* data, size_t words, bool zero, hipStream_t s) {
    hipLaunchKernelGGL(mfma_probe_fill_kernel, dim3(2048), dim3(256), 0, s, data, words, zero ? 1u : 0u);
    return hipGetLastError();
}

}  // namespace kleos_amd
