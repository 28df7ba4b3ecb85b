// Kernels of the MoE layer forward and their launchers.
//
// Two ways to run the same device functions:
//   * phased: one launch per phase (gate, slotting, up-projection, down-projection, combine);
//   * fused:  one persistent launch for the whole layer, which is what the reference's
//     moe::forward is (csrc/include/kleos/moe/moe.cuh:77-144). The reference dedicates one block
//     to an in-kernel "OS" (scheduler + subscriber warps, os/os.cuh:32-216, os/scheduler.cuh,
//     os/subscriber.cuh) that hands 128-byte task descriptors to processor blocks through
//     doorbells and is driven by NVSHMEM signal flags. Here every workgroup is a processor and the
//     scheduler is a handful of device-scope atomic counters: a ticket counter per XCD queue over
//     a statically ordered tile list, and one readiness counter per (expert, row block) that
//     releases the down-projection tiles once all up-projection tiles of that block are stored
//     (the reference's tQS counter + notifyNext, os/processor/processor.cuh:516-636,719-729).
#include "kernels.hpp"

#include <type_traits>

#include "combine.hpp"
#include "device_common.hpp"
#include "expert_gemm.hpp"
#include "gate.hpp"

namespace kleos_amd {

namespace {

constexpr int kXcds = 8;
// expert GEMM tile of the bf16 path
constexpr int kBM = 256, kBN = 256;
constexpr int kWavesM = 2, kWavesN = 4;   // wavefront grid over the tile
constexpr int kGemmThreads = kWavesM * kWavesN * kWave;

// Tile shape and workgroup size of the expert projections per Element type. The workgroup size is
// also that of the persistent kernel, whose other phases run on groups of its wavefronts.
template <typename T> struct TileShape;
template <> struct TileShape<bf16_t> { static constexpr int BM = kBM, BN = kBN, kThreads = kGemmThreads; };
template <> struct TileShape<float> { static constexpr int BM = kF32Tile, BN = kF32Tile, kThreads = 256; };
constexpr int kPhaseThreads = 256;   // gate, slot and combine kernels of the phased mode

template <typename T>
constexpr int gemm_smem_bytes() {
    if constexpr (sizeof(T) == 2) return gemm_bf16_smem_bytes<kBM, kBN>();
    else return gemm_f32_smem_bytes();
}

__host__ __device__ inline uint32_t ceil_div_u32(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

__device__ __forceinline__ uint32_t kept_rows(const LayerParams& p, uint32_t e) {
    // consumers clamp the routed count to the capacity (packet.cuh:85,112-113)
    const uint32_t c = p.expert_count[e];
    const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
    return c < cap ? c : cap;
}

// One output tile of an expert projection. kind 0: h1 = act(x_gathered * Wup^T + bup);
// kind 1: y = h1 * Wdown^T + bdown (identity activation, types.cuh:461).
template <typename T>
__device__ __forceinline__ void expert_tile(const LayerParams& p, uint32_t e, uint32_t kind,
                                            uint32_t mtile, uint32_t ntile, uint32_t rows,
                                            char* smem) {
    constexpr int BM = TileShape<T>::BM, BN = TileShape<T>::BN;
    const uint32_t row0 = mtile * BM, col0 = ntile * BN;
    const uint32_t m_valid = rows - row0 < uint32_t(BM) ? rows - row0 : uint32_t(BM);
    const uint32_t N = kind == 0 ? p.I : p.H, K = kind == 0 ? p.H : p.I;
    const uint32_t n_valid = N - col0 < uint32_t(BN) ? N - col0 : uint32_t(BN);
    const T* w = static_cast<const T*>(kind == 0 ? p.w_up : p.w_down) + size_t(e) * p.I * p.H + size_t(col0) * K;
    const T* bias = static_cast<const T*>(kind == 0 ? p.b_up : p.b_down) + size_t(e) * N + col0;
    const size_t row_base = size_t(e) * p.cap_rows + row0;
    if (kind == 0) {
        const T* a = static_cast<const T*>(p.x);
        const int32_t* idx = p.slot_token + row_base;
        T* c = static_cast<T*>(p.h1) + row_base * p.I + col0;
        auto run = [&](auto act_tag) {
            constexpr int ACT = decltype(act_tag)::value;
            if constexpr (sizeof(T) == 2)
                gemm_tile_bf16<ACT, BM, BN, kWavesM, kWavesN, 0>(a, idx, p.H, m_valid, w, K, n_valid, bias, c, p.I, K, smem);
            else
                gemm_tile_f32<ACT>(a, idx, p.H, m_valid, w, K, n_valid, bias, c, p.I, K, smem);
        };
        if (p.act == 0) run(std::integral_constant<int, 0>{});
        else run(std::integral_constant<int, 1>{});
    } else {
        const T* a = static_cast<const T*>(p.h1) + row_base * p.I;
        T* c = static_cast<T*>(p.y) + row_base * p.H + col0;
        if constexpr (sizeof(T) == 2)
            gemm_tile_bf16<2, BM, BN, kWavesM, kWavesN, 1>(a, nullptr, p.I, m_valid, w, K, n_valid, bias, c, p.H, K, smem);
        else
            gemm_tile_f32<2>(a, nullptr, p.I, m_valid, w, K, n_valid, bias, c, p.H, K, smem);
    }
}

// ------------------------------------------------------------------------------------ phased
template <typename T, int NG>
__global__ __launch_bounds__(kPhaseThreads) void gate_kernel(const LayerParams p) {
    __shared__ float smem[gate_smem_floats<NG>()];
    gate_tile<T, NG>(p, blockIdx.x, true, smem);
}

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

// Workgroup -> (expert, row block, column block). Consecutive workgroup ids land on consecutive
// XCDs, so expert e is pinned to XCD e % 8: all tiles that share its weights and its activation
// rows meet in one L2. Row blocks vary fastest so that the tiles re-reading one weight tile run
// together.
template <typename T>
__global__ __launch_bounds__(TileShape<T>::kThreads) void expert_gemm_kernel(const LayerParams p, uint32_t kind,
                                                               uint32_t tiles_m, uint32_t tiles_n) {
    extern __shared__ __attribute__((aligned(16))) char gemm_smem[];
    const uint32_t per_expert = tiles_m * tiles_n;
    uint32_t e, rem;
    if (p.E % kXcds == 0) {
        const uint32_t xcd = blockIdx.x % kXcds, j = blockIdx.x / kXcds;
        e = xcd + kXcds * (j / per_expert);
        rem = j % per_expert;
    } else {
        e = blockIdx.x / per_expert;
        rem = blockIdx.x % per_expert;
    }
    const uint32_t mtile = rem % tiles_m, ntile = rem / tiles_m;
    const uint32_t rows = kept_rows(p, e);
    if (mtile * TileShape<T>::BM >= rows) return;
    expert_tile<T>(p, e, kind, mtile, ntile, rows, gemm_smem);
}

template <typename T>
__global__ __launch_bounds__(kPhaseThreads) void combine_kernel(const LayerParams p) {
    const uint32_t token = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (token < p.S) combine_token<T>(p, token);
}

// ------------------------------------------------------------------------------------ fused
// Scheduler words (uint32), all in p.sched:
//   [0..2]                 grid-barrier arrival counters, monotonically increasing across launches
//   [8..15]                ticket counter of each XCD queue
//   [16 .. 16+E*mt_max)    readiness: up-projection tiles stored per (expert, row block)
//   [4]                    set to non-zero by a workgroup whose bounded wait expired
constexpr uint32_t kSchedBar = 0, kSchedError = 4, kSchedTicket = 8, kSchedReady = 16;
// Every wait in the persistent kernel is bounded so that the grid always drains: after this many
// ticks of the 100 MHz wall clock a waiter records an error and proceeds.
constexpr unsigned long long kWaitTicks = 300000000ull;   // 3 s
// LDS header of the expert phase (bytes)
constexpr size_t kLdsMt = 512, kLdsQueue = 128, kLdsSeg = 8 * (2 * 16 * kMaxGateGroups);
constexpr size_t kFusedLdsHeader = kLdsMt + kLdsQueue + kLdsSeg;

struct Segment {
    uint16_t expert;
    uint8_t kind;
    uint8_t pad;
    uint32_t start;     // first ticket of the segment inside its queue
};

// Spins (thread 0 only) until pred() holds or the wait bound expires.
template <typename Pred>
__device__ __forceinline__ void bounded_wait(uint32_t* sched, Pred&& pred) {
    if (pred()) return;
    const unsigned long long t0 = wall_clock64();
    while (!pred()) {
        __builtin_amdgcn_s_sleep(2);
        if (wall_clock64() - t0 > kWaitTicks) {
            atomic_store_relaxed(sched + kSchedError, 1u);
            return;
        }
    }
}

__device__ __forceinline__ void grid_barrier(uint32_t* sched, uint32_t which, uint32_t target) {
    uint32_t* ctr = sched + kSchedBar + which;
    __syncthreads();
    if (threadIdx.x == 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        atomic_add_agent(ctr, 1u);
        bounded_wait(sched, [&] { return int32_t(atomic_load_relaxed(ctr) - target) >= 0; });
    }
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

template <typename T, int NG>
__global__ __launch_bounds__(TileShape<T>::kThreads) void fused_kernel(const LayerParams p, uint32_t barrier_base,
                                                                      uint32_t mt_max, uint32_t lag) {
    static_assert(sizeof(Segment) == 8, "segment table sizing");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int BM = TileShape<T>::BM, BN = TileShape<T>::BN;
    constexpr uint32_t kThreads = TileShape<T>::kThreads;
    constexpr uint32_t kWaves = kThreads / kWave, kGroups = kThreads / 256;
    const uint32_t tid = threadIdx.x, wave = tid >> 6, group = tid >> 8;
    const uint32_t nwg = gridDim.x;
    uint32_t* sched = p.sched;
    unsigned long long* stamp = p.stamps + size_t(blockIdx.x) * 8;
    if (tid == 0) stamp[0] = wall_clock64();

    // ---- phase 0: gate. Workgroup 0 also resets this launch's tickets and readiness counters;
    // nothing reads them before the second barrier.
    if (blockIdx.x == 0) {
        for (uint32_t i = tid; i < kXcds + p.E * mt_max; i += kThreads) sched[kSchedTicket + i] = 0u;
    }
    for (uint32_t t0 = blockIdx.x * kGroups; t0 < p.n_gate_tiles; t0 += nwg * kGroups)
        gate_tile<T, NG>(p, t0 + group, t0 + group < p.n_gate_tiles,
                         reinterpret_cast<float*>(smem) + group * gate_smem_floats<NG>());
    if (tid == 0) stamp[1] = wall_clock64();
    grid_barrier(sched, 0, barrier_base + nwg);
    if (tid == 0) stamp[2] = wall_clock64();

    // ---- phase 1: slots in token order
    {
        uint32_t* base = reinterpret_cast<uint32_t*>(smem) + wave * p.E;
        for (uint32_t t0 = blockIdx.x * kWaves; t0 < p.n_gate_tiles; t0 += nwg * kWaves)
            slot_tile(p, t0 + wave, t0 + wave < p.n_gate_tiles, base);
        uint32_t* other = p.super_count + size_t((p.epoch & 1u) ^ 1u) * p.n_super * p.E;
        for (uint32_t i = blockIdx.x * kThreads + tid; i < p.n_super * p.E; i += nwg * kThreads) other[i] = 0u;
    }
    if (tid == 0) stamp[3] = wall_clock64();
    grid_barrier(sched, 1, barrier_base + nwg);
    if (tid == 0) stamp[4] = wall_clock64();

    // ---- phase 2: expert tiles from per-XCD ticket queues
    // LDS map: row blocks per expert | queue starts, totals, task | segments | GEMM tile
    uint16_t* s_mt = reinterpret_cast<uint16_t*>(smem);                         // [E], E <= 256
    uint32_t* s_qseg = reinterpret_cast<uint32_t*>(smem + kLdsMt);              // [9] first segment of each queue
    uint32_t* s_qtot = s_qseg + 16;                                             // [8] tickets in each queue
    uint32_t* s_task = s_qtot + 8;                                              // [5] expert, kind, mtile, ntile, stolen (kind 2 = stop)
    Segment* s_seg = reinterpret_cast<Segment*>(smem + kLdsMt + kLdsQueue);     // at most 2*E segments
    char* s_gemm = smem + kFusedLdsHeader;
    const uint32_t tn_up = ceil_div_u32(p.I, BN), tn_down = ceil_div_u32(p.H, BN);

    for (uint32_t e = tid; e < p.E; e += kThreads) s_mt[e] = uint16_t(ceil_div_u32(kept_rows(p, e), BM));
    __syncthreads();
    if (tid == 0) {
        uint32_t nseg = 0;
        for (uint32_t q = 0; q < kXcds; ++q) {
            s_qseg[q] = nseg;
            const uint32_t nq = q < p.E ? (p.E - q + kXcds - 1) / kXcds : 0u;   // experts q, q+8, ...
            uint32_t ticket = 0;
            // up-projection of expert i, then down-projection of expert i - lag: a down tile is
            // handed out only after `lag` further experts' worth of tickets, by which time the
            // up tiles it depends on have normally been stored.
            for (uint32_t i = 0; i < nq + lag; ++i) {
                if (i < nq) {
                    const uint32_t e = q + kXcds * i;
                    s_seg[nseg++] = Segment{uint16_t(e), 0, 0, ticket};
                    ticket += uint32_t(s_mt[e]) * tn_up;
                }
                if (i >= lag) {
                    const uint32_t e = q + kXcds * (i - lag);
                    s_seg[nseg++] = Segment{uint16_t(e), 1, 0, ticket};
                    ticket += uint32_t(s_mt[e]) * tn_down;
                }
            }
            s_qtot[q] = ticket;
        }
        s_qseg[kXcds] = nseg;
    }
    __syncthreads();

    // The XCD this workgroup really runs on (hardware register XCC_ID): expert e's tiles are queued
    // on XCD e % 8, so that its weights, its gathered rows and the h1 rows handed from its
    // up-projection to its down-projection all live in one L2.
    const uint32_t xcd = __builtin_amdgcn_s_getreg((3 << 11) | 20) & (kXcds - 1);
    uint32_t q_off = 0;   // queues already found empty, starting from this workgroup's own XCD
    for (;;) {
        if (tid == 0) {
            uint32_t kind = 2, e = 0, mtile = 0, ntile = 0, stolen = 0;
            while (q_off < kXcds) {
                const uint32_t q = (xcd + q_off) % kXcds;
                // cheap pre-check keeps exhausted queues from being hammered
                if (s_qtot[q] == 0) { ++q_off; continue; }
                const uint32_t ticket = atomic_add_agent(sched + kSchedTicket + q, 1u);
                if (ticket >= s_qtot[q]) { ++q_off; continue; }
                uint32_t s = s_qseg[q];
                const uint32_t s_end = s_qseg[q + 1];
                while (s + 1 < s_end && s_seg[s + 1].start <= ticket) ++s;
                e = s_seg[s].expert;
                kind = s_seg[s].kind;
                const uint32_t local = ticket - s_seg[s].start;
                mtile = local % s_mt[e];
                ntile = local / s_mt[e];
                stolen = q_off != 0;
                break;
            }
            if (kind == 1) {
                // wait until every up-projection tile of this row block is stored
                const uint32_t* ready = sched + kSchedReady + e * mt_max + mtile;
                bounded_wait(sched, [&] { return atomic_load_relaxed(ready) >= tn_up; });
            }
            s_task[0] = e; s_task[1] = kind; s_task[2] = mtile; s_task[3] = ntile; s_task[4] = stolen;
        }
        __syncthreads();
        const uint32_t e = s_task[0], kind = s_task[1], mtile = s_task[2], ntile = s_task[3];
        if (kind == 2) break;
        // h1 rows written on this XCD are current in its L2 and the down-projection reads them
        // past the L1; rows written on another XCD (a tile taken from a foreign queue) need the
        // device-scope acquire, which drops this XCD's stale L2 lines.
        if (kind == 1 && (s_task[4] || sizeof(T) != 2)) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        expert_tile<T>(p, e, kind, mtile, ntile, kept_rows(p, e), s_gemm);
        __syncthreads();   // all stores of the tile issued; also protects s_task
        if (kind == 0 && tid == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            atomic_add_agent(sched + kSchedReady + e * mt_max + mtile, 1u);
        }
    }
    if (tid == 0) stamp[5] = wall_clock64();
    grid_barrier(sched, 2, barrier_base + nwg);
    if (tid == 0) stamp[6] = wall_clock64();

    // ---- phase 3: combine, one token per wavefront
    for (uint32_t token = blockIdx.x * kWaves + wave; token < p.S; token += nwg * kWaves) combine_token<T>(p, token);
    __syncthreads();
    if (tid == 0) stamp[7] = wall_clock64();
}

template <typename T, int NG>
size_t fused_smem_bytes(uint32_t E) {
    size_t need = kFusedLdsHeader + gemm_smem_bytes<T>();
    const size_t gate = (TileShape<T>::kThreads / 256) * gate_smem_floats<NG>() * sizeof(float);
    const size_t slots = (TileShape<T>::kThreads / kWave) * size_t(E) * sizeof(uint32_t);
    if (gate > need) need = gate;
    if (slots > need) need = slots;
    return need;
}

int gate_groups(uint32_t E) {
    const uint32_t g = ceil_div_u32(E, 16);
    if (g <= 1) return 1;
    if (g <= 2) return 2;
    if (g <= 4) return 4;
    if (g <= 8) return 8;
    return 16;
}

template <typename F>
hipError_t dispatch_groups(uint32_t E, F&& f) {
    switch (gate_groups(E)) {
        case 1: return f(std::integral_constant<int, 1>{});
        case 2: return f(std::integral_constant<int, 2>{});
        case 4: return f(std::integral_constant<int, 4>{});
        case 8: return f(std::integral_constant<int, 8>{});
        default: return f(std::integral_constant<int, 16>{});
    }
}

}  // namespace

const char* unsupported_reason(uint32_t E, uint32_t k) {
    (void)k;
    if (E > 16 * kMaxGateGroups) return "num_experts > 256 is not supported by the gate kernel of this build";
    return nullptr;
}

uint32_t sched_error_word() { return kSchedError; }

#ifdef KLEOS_TRACE
extern "C" int kleos_trace_attach(unsigned long long* device_buffer) {
    return int(hipMemcpyToSymbol(HIP_SYMBOL(g_trace), &device_buffer, sizeof(device_buffer)));
}
#endif

size_t sched_words(uint32_t E, uint32_t cap_rows) {
    return kSchedReady + size_t(E) * ceil_div_u32(cap_rows, 64) + 64;
}

hipError_t launch_gate(const LayerParams& p, int dtype, hipStream_t s) {
    return dispatch_groups(p.E, [&](auto ng) {
        constexpr int NG = decltype(ng)::value;
        if (dtype == 2) hipLaunchKernelGGL((gate_kernel<bf16_t, NG>), dim3(p.n_gate_tiles), dim3(kPhaseThreads), 0, s, p);
        else hipLaunchKernelGGL((gate_kernel<float, NG>), dim3(p.n_gate_tiles), dim3(kPhaseThreads), 0, s, p);
        return hipGetLastError();
    });
}

hipError_t launch_slots(const LayerParams& p, hipStream_t s) {
    const uint32_t grid = ceil_div_u32(p.n_gate_tiles, 4);
    hipLaunchKernelGGL(slot_kernel, dim3(grid), dim3(kPhaseThreads), 4 * p.E * sizeof(uint32_t), s, p);
    return hipGetLastError();
}

hipError_t launch_expert_gemm(const LayerParams& p, int dtype, int kind, hipStream_t s) {
    const uint32_t N = kind == 0 ? p.I : p.H;
    auto go = [&](auto tag) {
        using T = decltype(tag);
        const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
        const uint32_t tiles_m = ceil_div_u32(cap, TileShape<T>::BM), tiles_n = ceil_div_u32(N, TileShape<T>::BN);
        const uint32_t grid = p.E * tiles_m * tiles_n;
        auto kernel = expert_gemm_kernel<T>;
        // more than 64 KB of dynamic LDS has to be asked for explicitly
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, gemm_smem_bytes<T>());
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(TileShape<T>::kThreads), gemm_smem_bytes<T>(), s, p,
                           uint32_t(kind), tiles_m, tiles_n);
        return hipGetLastError();
    };
    return dtype == 2 ? go(bf16_t{}) : go(float{});
}

hipError_t launch_combine(const LayerParams& p, int dtype, hipStream_t s) {
    const uint32_t grid = ceil_div_u32(p.S, 4);
    if (dtype == 2) hipLaunchKernelGGL((combine_kernel<bf16_t>), dim3(grid), dim3(kPhaseThreads), 0, s, p);
    else hipLaunchKernelGGL((combine_kernel<float>), dim3(grid), dim3(kPhaseThreads), 0, s, p);
    return hipGetLastError();
}

hipError_t plan_fused(const LayerParams& p, int dtype, int num_cus, FusedPlan* plan) {
    return dispatch_groups(p.E, [&](auto ng) -> hipError_t {
        constexpr int NG = decltype(ng)::value;
        auto go = [&](auto tag) -> hipError_t {
            using T = decltype(tag);
            auto kernel = fused_kernel<T, NG>;
            const size_t smem = fused_smem_bytes<T, NG>(p.E);
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
            if (err != hipSuccess) return err;
            int occ = 0;
            err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, TileShape<T>::kThreads, smem);
            if (err != hipSuccess) return err;
            if (occ < 1) return hipErrorLaunchOutOfResources;
            if (occ > 2) occ = 2;
            // every workgroup must be resident at once: the kernel holds grid-wide barriers
            plan->nwg = uint32_t(num_cus) * uint32_t(occ);
            plan->smem = smem;
            const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
            plan->mt_max = ceil_div_u32(cap, TileShape<T>::BM);
            // tickets that separate an expert's up tiles from its down tiles: about one wave of
            // the resident workgroups of a queue
            const uint32_t tiles_per_expert = plan->mt_max * ceil_div_u32(p.I, TileShape<T>::BN);
            plan->lag = ceil_div_u32(ceil_div_u32(plan->nwg, kXcds), tiles_per_expert ? tiles_per_expert : 1u);
            if (plan->lag < 1) plan->lag = 1;
            plan->kernel = reinterpret_cast<const void*>(kernel);
            plan->threads = TileShape<T>::kThreads;
            return hipSuccess;
        };
        return dtype == 2 ? go(bf16_t{}) : go(float{});
    });
}

hipError_t launch_fused(const LayerParams& p, const FusedPlan& plan, uint32_t fused_seq, hipStream_t s) {
    // arrivals recorded on the barrier counters by earlier fused launches (mod 2^32)
    uint32_t barrier_base = fused_seq * plan.nwg;
    uint32_t mt_max = plan.mt_max, lag = plan.lag;
    LayerParams pc = p;
    void* args[] = {&pc, &barrier_base, &mt_max, &lag};
    return hipLaunchKernel(plan.kernel, dim3(plan.nwg), dim3(plan.threads), args, plan.smem, s);
}

}  // namespace kleos_amd
