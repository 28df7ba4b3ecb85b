// Kernels of the MoE layer forward and their launchers, as templates over the Element type. Every
// Element type is instantiated in a translation unit of its own (kernels_f32.hip, kernels_bf16.hip,
// kernels_f16.hip: they compile side by side); kernels.hip holds what does not depend on the type.
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
//     When the queues hold equal work the same tile list is walked without tickets: each XCD's
//     workgroups stride through it by a rank they take at the start (the static schedule, chosen
//     per launch inside the kernel); the readiness counters stay, and since a queue lists all its
//     up-projection tiles before its down-projection tiles they are normally complete long before
//     they are looked at.
#pragma once
#include "kernels.hpp"

#include <type_traits>

#include "combine.hpp"
#include "device_common.hpp"
#include "expert_gemm.hpp"
#include "gate.hpp"

namespace kleos_amd {

namespace {

constexpr int kXcds = 8;
// Expert GEMM configuration of the bf16 / fp16 path: 256 x 256 tile (an expert's whole capacity of
// 256 rows at the headline shape, so its weights stream from HBM exactly once), 4 x 2 wavefronts of
// 64 x 128 (two per SIMD), K slices of 64 (whole 128-byte lines of every row) through two 64 KB
// stages, loads two slices ahead, a slice's loads shared out 4 + 4 over two quarters of a slice's
// matrix instructions, which are the 16x16x32 ones (see Gemm16: they draw less power, and power is
// what bounds these kernels: 292 against 298 us per forward at the headline shape with 32x32x16,
// 3.16 against 3.28 ms at the 8-expert shape with hidden size 4096; with them 4 + 4 beats 3 + 3 + 2,
// which was the better split for the 32x32x16 instructions, 291 against 298 us).
// (Measured against it on MI355X, none faster: K slices of 32 through four stages, 2 x 2 wavefronts
// of 128 x 128 with the accumulators in AGPRs, weight slices of 64 through three slots with
// activation half slices of 32 through three, the 128 x 256 tile of variant 1. 2 x 4 wavefronts
// of 128 x 64: 305.0 against 299.8 us per forward at the headline shape, 158.3 against 155.7 at
// the 16-expert shape, whose tiles are all full; with four rows of wavefronts those whose rows do
// not exist in a tile also come in steps of 64 rows.)
// Variant 1, for layers whose experts hold at most 128 rows (many small experts): a 128 x 256 tile
// wastes no matrix work and no activation loads on rows that do not exist, and its smaller stages
// leave room for a third one (measured on the 256-expert top-8 shape: 3.7 ms against 4.6 ms).
// Variant 2, for layers whose experts hold at least four row blocks (few large experts: every
// weight tile is shared by several workgroups through L2, loads return quickly and the matrix work
// dominates): the tile of variant 0 on 2 x 4 wavefronts of 128 x 64 (3.53 against 3.57 ms with 4 x 2
// at the 8-expert shape with hidden size 4096), the loads two slices ahead like variant 0 and shared
// out 4 + 4 over two quarters of a slice (both projections of that shape on random data, 32x32x16
// instructions: 3.95 ms against 4.11 with the loads one slice ahead, all behind the first K step, and 4.18
// two slices ahead all at once).
// Variants 0 and 1 load their weight rows non-temporally (headline 378 against 390 us per forward,
// the 16-expert shape 192 against 196, the 256-expert shape 3.43 against 3.48 ms); variant 2, whose
// weight tiles are shared by eight workgroups and more, does not (4.06 against 4.01 ms with it).
// (The choices below can be overridden on the compiler's command line for measurements.)
#ifndef KLEOS_TUNE_V0_SPREAD
#define KLEOS_TUNE_V0_SPREAD 1       // variant 0: loads of a slice issued 4 + 4 over two quarters of a slice (2: 3 + 3 + 2)
#endif
#ifndef KLEOS_TUNE_V2_SPREAD
#define KLEOS_TUNE_V2_SPREAD 1       // variant 2: two slices ahead, 4 + 4 over two quarters of a slice; -1: one slice ahead
#endif
#ifndef KLEOS_TUNE_ZERO_PAD
#define KLEOS_TUNE_ZERO_PAD 1      // activation rows past an expert's last row read zeros instead of its last row
#endif
#ifndef KLEOS_TUNE_HALVED_TAIL
#define KLEOS_TUNE_HALVED_TAIL 1   // dynamic schedule: the last down-projection tiles of a queue as halves of 128 rows
#endif
#ifndef KLEOS_TUNE_MIXED_HEIGHTS
#define KLEOS_TUNE_MIXED_HEIGHTS 1   // variant 2: 128-row tiles for last row blocks of at most 128 rows
#endif
#ifndef KLEOS_TUNE_MI
#define KLEOS_TUNE_MI 16           // matrix-core tile of the expert GEMM: 16 (16x16x32 instructions) or 32 (32x32x16)
#endif
#ifndef KLEOS_TUNE_MI_V0
#define KLEOS_TUNE_MI_V0 16        // the same for variant 0 (switchable apart: its tiles are the ones bound by their loads)
#endif
#ifndef KLEOS_TUNE_V1_STREAM_OUT
#define KLEOS_TUNE_V1_STREAM_OUT 1 // variant 1 (many small experts) stores its intermediate and output rows non-temporally
#endif
#ifndef KLEOS_TUNE_V0_RELEASE
#define KLEOS_TUNE_V0_RELEASE 1    // where variant 0 frees a slice's stage and issues the loads behind it (Gemm16's RELEASE)
#endif
#ifndef KLEOS_TUNE_V2_RELEASE
#define KLEOS_TUNE_V2_RELEASE 2    // the same for variant 2
#endif
template <typename E, int V>
using GemmCfg = std::conditional_t<V == 0, Gemm16<E, 256, 256, 4, 2, 64, 2, true, true, KLEOS_TUNE_V0_SPREAD, KLEOS_TUNE_MI_V0, KLEOS_TUNE_V0_RELEASE>,
                std::conditional_t<V == 1, Gemm16<E, 128, 256, 2, 4, 64, 3, true, false, 0, KLEOS_TUNE_MI, 0, (KLEOS_TUNE_V1_STREAM_OUT != 0)>,
                                   Gemm16<E, 256, 256, 2, 4, 64, 2, false, (KLEOS_TUNE_V2_SPREAD >= 0), (KLEOS_TUNE_V2_SPREAD >= 0 ? KLEOS_TUNE_V2_SPREAD : 0), KLEOS_TUNE_MI,
                                          KLEOS_TUNE_V2_RELEASE>>>;
// Layers of variant 2 mix two tile heights inside one launch: the last row block of an expert, when
// it holds at most 128 rows, goes to a 128 x 256 tile (three stages, loads two slices ahead of the
// slice being worked on) instead of a 256-row tile whose lower half would multiply rows that do
// not exist. The blocks keep their 256-row spacing in h1 and y; only the tile that works on them
// differs. (The K order of every output element is the same in both tiles: same slices, same
// matrix instruction, so which tile computed a row does not show in its bits.)
template <typename E, int V>
using NarrowCfg = Gemm16<E, 128, 256, 2, 4, 64, 3, false, false, 0, KLEOS_TUNE_MI>;
template <typename G> struct TypeTag { using type = G; };   // a type handed to a generic lambda
template <typename T, int V> constexpr bool kMixedHeights = sizeof(T) == 2 && V == 2 && KLEOS_TUNE_MIXED_HEIGHTS != 0;
constexpr uint32_t kNarrowTileRows = 128;
// What the padding rows of an expert tile read: zeros, as long as the inner dimension is no longer than this.
constexpr int kZeroRowElems = 16384;
static __device__ __attribute__((aligned(256))) const elem16_t g_zero_row[kZeroRowElems] = {};
constexpr int kBN = 256;
constexpr int kGemmThreads = GemmCfg<bf16_t, 0>::kThreads;
static_assert(NarrowCfg<bf16_t, 2>::kThreads == kGemmThreads, "both tile heights run on the same workgroup");
static_assert(GemmCfg<bf16_t, 1>::kThreads == kGemmThreads && GemmCfg<bf16_t, 2>::kThreads == kGemmThreads,
              "all variants share the workgroup size");
constexpr uint32_t kNarrowRows = 128;   // variant 1 when no expert can hold more rows than this
constexpr uint32_t kSharedRows = 1024;  // variant 2 when every expert can hold at least this many

// Tile shape and workgroup size of the expert projections per Element type. The workgroup size is
// also that of the persistent kernel, whose other phases run on groups of its wavefronts.
template <typename T, int V = 0> struct TileShape {
    static_assert(sizeof(T) == 2);
    static constexpr int BM = V == 1 ? 128 : 256, BN = kBN, kThreads = kGemmThreads, kPerCu = 1;
};
template <int V> struct TileShape<float, V> { static constexpr int BM = kF32Tile, BN = kF32Tile, kThreads = 256, kPerCu = 1; };
template <int V> struct TileShape<tf32_t, V> : TileShape<float, V> {};
constexpr int kPhaseThreads = 256;   // gate, slot and combine kernels of the phased mode

template <typename T, int V>
constexpr int gemm_smem_bytes() {
    if constexpr (kMixedHeights<T, V>)
        return GemmCfg<T, V>::kSmemBytes > NarrowCfg<T, V>::kSmemBytes ? GemmCfg<T, V>::kSmemBytes : NarrowCfg<T, V>::kSmemBytes;
    else if constexpr (sizeof(T) == 2) return GemmCfg<T, V>::kSmemBytes;
    else return gemm_f32_smem_bytes();
}
constexpr int kPhasedGemmHeader = 128;
constexpr int kStampWords = 16;         // per-workgroup phase stamps [0..7] and scheduler statistics [8..15]   // task broadcast slot in front of the GEMM stages

__host__ __device__ inline uint32_t ceil_div_u32(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// kCoherent: the counts were written earlier in the same launch (persistent kernel).
template <bool kCoherent>
__device__ __forceinline__ uint32_t kept_rows(const LayerParams& p, uint32_t e) {
    // consumers clamp the routed count to the capacity (packet.cuh:85,112-113)
    const uint32_t c = kCoherent ? load_coherent(p.expert_count + e) : p.expert_count[e];
    const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
    return c < cap ? c : cap;
}

// ------------------------------------------------------------------------------------ scheduler state
// Scheduler words (uint32), all in p.sched. Counters that different workgroups hit at the same
// time sit on 128-byte lines of their own (kSchedLine words apart): atomics on one line serialise.
//   kSchedBar + 32 b              grid barrier b: groups that have arrived, monotonic across launches
//   kSchedGroup + 32 (8 b + g)    grid barrier b: arrivals of workgroup group g, monotonic
//   kSchedTicket + 32 q           ticket counter of XCD queue q
//   kSchedMembers + 32 (8 h + x)  workgroups of this launch that run on XCD x; h = launch parity
//   kSchedReady + e*mt_max + m    readiness: up-projection tiles stored per (expert, row block)
//   kSchedError                   set to non-zero by a workgroup whose bounded wait expired
constexpr uint32_t kSchedLine = 32;
constexpr uint32_t kSchedBar = 0, kSchedError = 4, kSchedTicket = 4 * kSchedLine,
                   kSchedGroup = 12 * kSchedLine, kSchedMembers = 44 * kSchedLine, kSchedReady = 60 * kSchedLine;
constexpr uint32_t kGridBarriers = 4;   // 0 gate, 1 slots, 2 experts, 3 inside the gate (between its product and its epilogue)
// schedule of the expert phase of the persistent kernel (the values of kleos_amd.h's KLEOS_SCHEDULE_*)
constexpr uint32_t kScheduleAuto = 0, kScheduleStatic = 2;   // anything else: dynamic
static_assert(kSchedBar + kGridBarriers * kSchedLine <= kSchedTicket, "barrier words");
static_assert(kSchedGroup + kGridBarriers * kXcds * kSchedLine <= kSchedMembers, "barrier group words");
static_assert(kSchedMembers + 2 * kXcds * kSchedLine <= kSchedReady, "member words");
// Every wait in the persistent kernel is bounded so that the grid always drains: after
// LayerParams::wait_ticks ticks of the 100 MHz wall clock (3 s unless the host says otherwise) a
// waiter records an error and proceeds.
// LDS header of the expert phase (bytes)
// rows kept per expert u32[Ep] | row blocks u16[Ep] | queue words (kLdsQueue bytes) | segments [2 Ep],
// with Ep = the expert count rounded up to 64, at least 256
constexpr size_t kLdsQueue = 256;
constexpr uint32_t kMaxExperts = 512;   // the header and the tiles of the narrow variant share 160 KB of LDS
__host__ __device__ inline uint32_t lds_experts(uint32_t E) { return E <= 256 ? 256u : (E + 63) / 64 * 64; }
__host__ __device__ inline size_t lds_queue_offset(uint32_t E) { return size_t(6) * lds_experts(E); }
__host__ __device__ inline size_t fused_lds_header(uint32_t E) { return lds_queue_offset(E) + kLdsQueue + size_t(16) * lds_experts(E); }

struct Segment {
    uint16_t expert;
    uint8_t kind;
    uint8_t pad;
    uint32_t start;     // first ticket of the segment inside its queue
};

// Spins (one thread) until pred() holds or `ticks` ticks of the wall clock have passed.
template <typename Pred>
__device__ __forceinline__ void bounded_wait(uint32_t* sched, unsigned long long ticks, Pred&& pred) {
    if (pred()) return;
    const unsigned long long t0 = wall_clock64();
    while (!pred()) {
        __builtin_amdgcn_s_sleep(2);
        if (wall_clock64() - t0 > ticks) {
            atomic_store_relaxed(sched + kSchedError, 1u);
            return;
        }
    }
}

// Grid-wide barrier number `which` of persistent launch number `seq` (launches counted from 0 on
// this arena) of a grid of `nwg` resident workgroups. Arrivals are counted in two levels, eight
// groups of workgroups (id mod 8) whose last member reports the group: a few dozen atomics land on
// each counter instead of one per workgroup on a single word, which is what a flat barrier spends
// most of its time on when everybody arrives together. All counters only ever grow, so nothing is
// reset between launches.
// `between()` is called by every thread after the workgroup has arrived and before it waits for the
// others: work that does not depend on what the other workgroups are still writing rides in the
// wait. The arrival and the wait are the business of the first lane of the last wavefront, so that
// the wavefronts `between` keeps busy (it may hold workgroup barriers) do not sit behind the
// arrival's trips to memory longer than they must.
// Every wavefront first waits for its own outstanding stores. Whatever another workgroup reads
// after the barrier was written through the L2 (store_through and the like), so a store that has
// been acknowledged is visible device-wide and the arrival needs no device-scope release, which
// would write the whole L2 back (measured: 2 us per barrier and 11-19 us per forward at the
// 64-expert shape, the other workgroups of the XCD slowed down included).
template <typename Between>
__device__ __forceinline__ void grid_barrier(uint32_t* sched, unsigned long long ticks, uint32_t which, uint32_t seq, uint32_t nwg,
                                             Between&& between) {
    wait_vmcnt<0>();
    __syncthreads();
    const bool leader = threadIdx.x == blockDim.x - kWave;
    if (leader) {
        const uint32_t g = blockIdx.x % kXcds;
        const uint32_t members = (nwg - g + kXcds - 1) / kXcds;
        uint32_t* all = sched + kSchedBar + which * kSchedLine;
        uint32_t* mine = sched + kSchedGroup + (which * kXcds + g) * kSchedLine;
        // (the workgroup-scope fences keep the compiler from moving memory operations across the
        // arrivals; the hardware side is the drained vmcnt above)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (atomic_add_agent(mine, 1u) + 1u == (seq + 1u) * members) {
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
            atomic_add_agent(all, 1u);
        }
    }
    between();
    if (leader) {
        const uint32_t groups = nwg < uint32_t(kXcds) ? nwg : uint32_t(kXcds);
        uint32_t* all = sched + kSchedBar + which * kSchedLine;
        const uint32_t target = (seq + 1u) * groups;
        bounded_wait(sched, ticks, [&] { return int32_t(atomic_load_relaxed(all) - target) >= 0; });
    }
    __syncthreads();
    // No device-scope acquire here either: it would invalidate the whole L2 of the XCD (tens of
    // microseconds of refetching per launch). What crosses workgroups after a barrier is read
    // with device-coherent loads instead; this only drops the CU's own L1.
    asm volatile("buffer_inv sc0" ::: "memory");
}

__device__ __forceinline__ void grid_barrier(uint32_t* sched, unsigned long long ticks, uint32_t which, uint32_t seq, uint32_t nwg) {
    grid_barrier(sched, ticks, which, seq, nwg, [] {});
}

// Tokens the gate routed to expert e in this launch, dropped ones included: the sum of the coarse
// count rows, which are complete once the gate phase has been released.
__device__ __forceinline__ uint32_t routed_count(const LayerParams& p, uint32_t e) {
    const uint32_t* super = p.super_count + size_t(p.epoch & 1u) * p.n_super * p.E;
    uint32_t total = 0;
    constexpr uint32_t kBatch = 16;
    for (uint32_t r0 = 0; r0 < p.n_super; r0 += kBatch) {
        uint32_t v[kBatch];
#pragma unroll
        for (uint32_t u = 0; u < kBatch; ++u)
            v[u] = load_coherent(super + size_t(r0 + u < p.n_super ? r0 + u : p.n_super - 1) * p.E + e);
#pragma unroll
        for (uint32_t u = 0; u < kBatch; ++u) total += r0 + u < p.n_super ? v[u] : 0u;
    }
    return total;
}

__device__ __forceinline__ bool balanced_or_forced(uint32_t policy, bool balanced) {
    return policy == kScheduleStatic || (policy == kScheduleAuto && balanced);
}

// One unit of expert work: an output tile of the up-projection (kind 0: h1 = act(x_gathered *
// Wup^T + bup)) or of the down-projection (kind 1: y = h1 * Wdown^T + bdown, identity activation,
// types.cuh:461). The reference's 128-byte Task descriptor (types.cuh:565-654) shrinks to this.
struct Task {
    uint32_t e, kind, mtile, ntile;
    uint32_t rows;      // rows the expert keeps (routed count clamped to the capacity)
    uint32_t foreign;   // taken from another XCD's queue: its h1 rows may sit in a different L2
    uint32_t dep;       // down tile: the readiness counter of its row block as seen when handed out
    uint32_t ready;     // down tile whose up-projection row block was already complete when handed out
    uint32_t narrow;    // goes to the 128-row tile (layers that mix tile heights): a row block of at most 128 rows, or one half of a row block
    uint32_t half;      // narrow tile that starts 128 rows into its row block (the second half of a halved block)
    uint32_t valid;
};
constexpr int kTaskWords = 12;

// Thread 0 publishes a task through LDS; every thread of the workgroup returns the same task.
// The barrier inside also separates the caller's previous and next use of the LDS.
__device__ __forceinline__ Task broadcast_task(uint32_t* s_task, const Task& mine) {
    if (threadIdx.x == 0) {
        s_task[0] = mine.e; s_task[1] = mine.kind; s_task[2] = mine.mtile; s_task[3] = mine.ntile;
        s_task[4] = mine.foreign; s_task[5] = mine.ready; s_task[6] = mine.valid; s_task[7] = mine.rows;
        s_task[8] = mine.dep; s_task[9] = mine.narrow; s_task[10] = mine.half;
    }
    __syncthreads();
    Task t;
    t.e = s_task[0]; t.kind = s_task[1]; t.mtile = s_task[2]; t.ntile = s_task[3];
    t.foreign = s_task[4]; t.ready = s_task[5]; t.valid = s_task[6]; t.rows = s_task[7];
    t.dep = s_task[8]; t.narrow = s_task[9]; t.half = s_task[10];
    return t;
}

template <typename T>
struct TileOperands {
    const T* a; const int32_t* idx; const T* w; const T* bias; T* c;
    uint32_t lda, ldc, K, m_valid, n_valid, act;
};

template <typename T, int V>
__device__ __forceinline__ TileOperands<T> tile_operands(const LayerParams& p, const Task& t) {
    constexpr int BM = TileShape<T, V>::BM, BN = TileShape<T, V>::BN;
    TileOperands<T> o;
    const uint32_t rows = t.rows;
    const uint32_t row0 = t.mtile * BM + t.half * kNarrowTileRows, col0 = t.ntile * BN;
    const uint32_t N = t.kind == 0 ? p.I : p.H;
    const uint32_t height = t.narrow ? kNarrowTileRows : uint32_t(BM);
    o.K = t.kind == 0 ? p.H : p.I;
    o.m_valid = rows - row0 < height ? rows - row0 : height;
    o.n_valid = N - col0 < uint32_t(BN) ? N - col0 : uint32_t(BN);
    o.w = static_cast<const T*>(t.kind == 0 ? p.w_up : p.w_down) + size_t(t.e) * p.I * p.H + size_t(col0) * o.K;
    o.bias = static_cast<const T*>(t.kind == 0 ? p.b_up : p.b_down) + size_t(t.e) * N + col0;
    const size_t row_base = size_t(t.e) * p.cap_rows + row0;
    if (t.kind == 0) {
        o.a = static_cast<const T*>(p.x); o.idx = p.slot_token + row_base; o.lda = p.H;
        o.c = static_cast<T*>(p.h1) + row_base * p.I + col0; o.ldc = p.I; o.act = p.act;
    } else {
        o.a = static_cast<const T*>(p.h1) + row_base * p.I; o.idx = nullptr; o.lda = p.I;
        o.act = 2;
        if constexpr (sizeof(T) == 2) {   // the tile's piece of y: cap_rows rows of kOutPiece columns
            static_assert(BN == int(kOutPiece));
            o.c = static_cast<T*>(p.y) + y_offset(t.e, row0, col0, p.cap_rows, p.H, sizeof(T)); o.ldc = kOutPiece;
        } else {
            o.c = static_cast<T*>(p.y) + row_base * p.H + col0; o.ldc = p.H;
        }
    }
    return o;
}

// Whether row block `mtile` of an expert with `rows` rows goes to the 128-row tile.
template <typename T, int V>
__device__ __forceinline__ uint32_t narrow_block(uint32_t rows, uint32_t mtile) {
    if constexpr (kMixedHeights<T, V>) return uint32_t(rows - mtile * uint32_t(TileShape<T, V>::BM) <= kNarrowTileRows);
    else return 0u;
}

// The K slice the tiles of expert e start with, out of k_tiles. Workgroups that run at the same time
// work on different experts; started at different slices, they read different column offsets of
// their 4 KB weight rows and their requests spread over the memory channels. All in step at one
// offset they queue on a few channels (measured on streaming reads of this shape: 4.8 against
// 6.3 TB/s). A function of the expert alone: the tiles of one expert still read the same activation
// and weight slices at the same time and share them through L2, and what a tile computes does
// not depend on the schedule or the launch mode.
__device__ __forceinline__ uint32_t first_k_slice(uint32_t e, uint32_t E, uint32_t k_tiles) {
    if (E >= k_tiles) return e % k_tiles;
    return e * (k_tiles / E);
}

// Readiness of a down-projection tile: all up-projection tiles of its (expert, row block) stored.
struct Readiness {
    uint32_t* sched;      // nullptr: no cross-tile dependencies inside this launch (phased mode)
    uint32_t mt_max, tn_up;
    unsigned long long ticks;   // bound of a wait for a row block
    __device__ __forceinline__ uint32_t* counter(const Task& t) const { return sched + kSchedReady + t.e * mt_max + t.mtile; }
    // A counter holds the stored tiles of the row block in its low half and, in its high half, how
    // many of them were stored by a workgroup on a foreign XCD (from whose L2 they were written back
    // to memory, while this XCD's L2 may still hold the rows as an earlier launch left them).
    static constexpr uint32_t kForeignUnit = 0x10000u;
    __device__ __forceinline__ bool complete(uint32_t v) const { return (v & 0xffffu) >= tn_up; }
};

// The expert phase of one workgroup: tiles from `next` until it runs dry. `next()` is called by
// every thread and returns the same task in all of them without ever blocking on a dependency;
// blocking happens here, after the workgroup has published its own finished tile, so that two
// workgroups can never wait on each other's unpublished results.
// `stats` (thread 0 only, may be null) accumulates 100 MHz ticks spent [0] fetching tasks,
// [1] waiting for a dependency, [2] publishing, and counts [3] tiles, [4] tiles handed out before
// their inputs were complete, [5] tiles taken from a foreign queue.
template <typename T, int V, typename Next>
__device__ __forceinline__ void expert_loop(const LayerParams& p, char* smem, uint32_t* s_task, const Readiness rd,
                                            unsigned long long* stats, Next&& next_raw) {
    const uint32_t tid = threadIdx.x;
    unsigned long long st_next = 0, st_wait = 0, st_pub = 0, n_tiles = 0, n_late = 0, n_foreign = 0;
    auto next = [&]() {
        const unsigned long long t0 = wall_clock64();
        const Task t = next_raw();
        st_next += wall_clock64() - t0;
        if (t.valid) { ++n_tiles; n_late += !t.ready; n_foreign += t.foreign; }
        return t;
    };
    auto wait_ready = [&](Task& t) {
        // only a down tile handed out before its inputs were complete gets here
        const unsigned long long t0 = wall_clock64();
        if (tid == 0) {
            uint32_t seen = t.dep;
            bounded_wait(rd.sched, rd.ticks, [&] { seen = atomic_load_relaxed(rd.counter(t)); return rd.complete(seen); });
            s_task[kTaskWords - 1] = seen;
        }
        __syncthreads();
        t.dep = s_task[kTaskWords - 1];
        st_wait += wall_clock64() - t0;
    };
    auto flush_stats = [&]() {
        if (stats && tid == 0) {
            stats[0] = st_next; stats[1] = st_wait; stats[2] = st_pub; stats[3] = n_tiles; stats[4] = n_late; stats[5] = n_foreign;
        }
    };
    auto acquire = [&](const Task& t) {
        // Before a down tile reads h1 rows that other workgroups of this launch wrote: rows written
        // on this XCD are current in its L2, so dropping this CU's L1 is enough; rows written on
        // another XCD need the device-scope acquire, which also drops this XCD's stale L2 lines.
        // The same holds for rows a foreign workgroup stored on behalf of this XCD's queue.
        if (!rd.sched || t.kind != 1) return;
        if (t.foreign || t.dep >= Readiness::kForeignUnit) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        else asm volatile("buffer_inv sc0" ::: "memory");
    };
    auto publish = [&](const Task& t) {
        // all stores of the tile are complete in every wavefront, and they were written through the
        // L2: the rows are visible to whoever may read them. Count the tile (the reference's tQS
        // increment, processor.cuh:719)
        if (rd.sched && t.kind == 0 && tid == 0) {
            const unsigned long long t0 = wall_clock64();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            atomic_add_agent(rd.counter(t), t.foreign ? 1u + Readiness::kForeignUnit : 1u);
            st_pub += wall_clock64() - t0;
        }
    };

    if constexpr (sizeof(T) == 2) {
        auto args_of = [&](const Task& t) {
            const TileOperands<T> o = tile_operands<T, V>(p, t);
            GemmTileArgs g;
            g.a_base = reinterpret_cast<const elem16_t*>(o.a); g.a_row_index = o.idx; g.a_rows = p.S;
            g.a_pad = KLEOS_TUNE_ZERO_PAD != 0 && o.K <= uint32_t(kZeroRowElems) ? g_zero_row : nullptr;
            g.b_base = reinterpret_cast<const elem16_t*>(o.w); g.bias = reinterpret_cast<const elem16_t*>(o.bias);
            g.c_base = reinterpret_cast<elem16_t*>(o.c);
            g.lda = o.lda; g.ldb = o.K; g.ldc = o.ldc; g.K = o.K; g.m_valid = o.m_valid; g.n_valid = o.n_valid;
            g.k_first = first_k_slice(t.e, p.E, o.K / uint32_t(GemmCfg<T, V>::kSliceK));
            g.act = o.act;
            return g;
        };
        static_assert(GemmCfg<T, V>::kSliceK == NarrowCfg<T, V>::kSliceK);
        // An up-projection tile whose stores are issued but which other workgroups have not been told
        // of yet (valid == 0: none). Its stores are known to be complete behind the first barrier of
        // the next tile's main loop, so it is counted from there, at no cost; it is counted at once,
        // behind a wait for the stores, when the workgroup is about to block or to leave.
        Task pending{};
        auto publish_now = [&]() {
            if (pending.valid) {
                wait_vmcnt<0>();
                __syncthreads();
                publish(pending);
                pending.valid = 0;
            }
        };
        // Tiles of one height, from `cur` on, as one pipeline across tiles; returns the first task
        // that is not of this height (or is not valid), with nothing of its own left unpublished and
        // every wavefront out of the LDS the tiles used.
        auto run = [&](auto gemm_tag, auto narrow_tag, Task cur) -> Task {
            using G = typename decltype(gemm_tag)::type;
            constexpr uint32_t kNarrow = decltype(narrow_tag)::value ? 1u : 0u;
            typename G::Tile cur_t;
            typename G::Acc acc;
            if (cur.kind == 1 && !cur.ready) wait_ready(cur);
            acquire(cur);
            int bias_slot = 0;
            G::begin(cur_t, args_of(cur), 0, bias_slot, smem);
            for (;;) {
                G::mainloop(cur_t, acc, smem, [&] { if (pending.valid) publish(pending); });
                pending.valid = 0;
                const Task nxt = next();   // its barrier: every wavefront has left the main loop
                G::finish(cur_t, acc, smem);
                if (rd.sched && cur.kind == 0) pending = cur;
                if (!nxt.valid || nxt.narrow != kNarrow) {
                    publish_now();
                    if (nxt.valid) __syncthreads();   // the other tile height lays the LDS out differently
                    return nxt;
                }
                cur = nxt;
                if (cur.kind == 1 && !cur.ready) {
                    publish_now();   // never wait while holding back a result of our own
                    wait_ready(cur);
                }
                acquire(cur);
                G::begin(cur_t, args_of(cur), G::next_stage0(cur_t), bias_slot ^= 1, smem);
            }
        };
        Task t = next();
        while (t.valid) {
            if constexpr (kMixedHeights<T, V>) {
                if (t.narrow) t = run(TypeTag<NarrowCfg<T, V>>{}, std::true_type{}, t);
                else t = run(TypeTag<GemmCfg<T, V>>{}, std::false_type{}, t);
            } else {
                t = run(TypeTag<GemmCfg<T, V>>{}, std::false_type{}, t);
            }
        }
        flush_stats();
    } else {
        for (;;) {
            Task t = next();
            if (!t.valid) break;
            if (t.kind == 1 && !t.ready) wait_ready(t);
            acquire(t);
            const TileOperands<T> o = tile_operands<T, V>(p, t);
            if (o.act == 0) gemm_tile_f32<0>(o.a, o.idx, p.S, o.lda, o.m_valid, o.w, o.K, o.n_valid, o.bias, o.c, o.ldc, o.K, smem);
            else if (o.act == 1) gemm_tile_f32<1>(o.a, o.idx, p.S, o.lda, o.m_valid, o.w, o.K, o.n_valid, o.bias, o.c, o.ldc, o.K, smem);
            else gemm_tile_f32<2>(o.a, o.idx, p.S, o.lda, o.m_valid, o.w, o.K, o.n_valid, o.bias, o.c, o.ldc, o.K, smem);
            wait_vmcnt<0>();   // the tile's stores, in every wavefront, before it is counted
            __syncthreads();
            publish(t);
        }
        flush_stats();
    }
}

// ------------------------------------------------------------------------------------ gate as a tiled product
// Logits of the 16-bit Elements with more than 64 experts: tiles of 128 tokens x 256 experts over a
// range of the hidden dimension, fp32 sums to p.gate_partial. Three stages of K slices (the gate
// weights come from L2, the activations stream from HBM once).
template <typename E>
using GateGemm = Gemm16<E, 128, 256, 2, 4, 64, 3, false, false>;
constexpr uint32_t kGateTileM = 128, kGateTileN = 256, kGateMaxSplits = 16;
static_assert(GateGemm<bf16_t>::kThreads == kGemmThreads, "the gate product runs on the workgroups of the expert phase");

__host__ __device__ inline uint32_t gate_gemm_tiles(const LayerParams& p) {
    return (p.S / kGateTileM) * ceil_div_u32(p.PX, kGateTileN) * p.gate_splits;
}

// Tiles first, first + stride, ... of the gate product. Every thread of the workgroup must call it.
template <typename T>
__device__ __forceinline__ void gate_gemm_phase(const LayerParams& p, char* smem, uint32_t first, uint32_t stride) {
    using G = GateGemm<T>;
    const uint32_t tiles_n = ceil_div_u32(p.PX, kGateTileN), splits = p.gate_splits;
    const uint32_t slices = p.H / uint32_t(G::kSliceK);
    typename G::Tile t;
    typename G::Acc acc;
    for (uint32_t tile = first; tile < gate_gemm_tiles(p); tile += stride) {
        // the ranges of one token block sit next to each other, so that they run at the same time
        const uint32_t split = tile % splits, rest = tile / splits;
        const uint32_t nb = rest % tiles_n, mb = rest / tiles_n;
        const uint32_t k0 = (slices * split) / splits, k1 = (slices * (split + 1)) / splits;
        GemmTileArgs g;
        g.a_base = static_cast<const elem16_t*>(p.x) + size_t(mb) * kGateTileM * p.H + size_t(k0) * G::kSliceK;
        g.a_row_index = nullptr; g.a_rows = p.S; g.a_pad = nullptr;
        g.b_base = static_cast<const elem16_t*>(p.wg) + size_t(nb) * kGateTileN * p.H + size_t(k0) * G::kSliceK;
        g.bias = static_cast<const elem16_t*>(p.wg);   // any readable 512 bytes: the sums take no bias
        g.c_base = nullptr;
        g.lda = p.H; g.ldb = p.H; g.ldc = 0; g.K = (k1 - k0) * G::kSliceK;
        g.k_first = 0;
        g.m_valid = kGateTileM;
        g.n_valid = p.PX - nb * kGateTileN < kGateTileN ? p.PX - nb * kGateTileN : kGateTileN;
        g.act = 2;
        __syncthreads();   // every wavefront has left the previous tile's epilogue staging
        if (k1 > k0) {
            G::begin(t, g, 0, 0, smem);
            G::mainloop(t, acc, smem);
            __syncthreads();
            float* out = p.gate_partial + (size_t(split) * p.S + size_t(mb) * kGateTileM) * p.PX + nb * kGateTileN;
            G::finish_partial(t, acc, smem, out, p.PX);
        }
    }
}

__host__ __device__ inline uint32_t gate_reduce_wave_words(const LayerParams& p);
// After the product: the 16-token tiles wg, wg + nwg, ... of the calling workgroup. Up to 256
// experts a tile goes to a group of four wavefronts (gate_reduce_group), above to a single one.
// Every thread of the workgroup must call it (workgroup barriers inside).
template <typename T, int NG>
__device__ __forceinline__ void gate_reduce_phase(const LayerParams& p, float* smem, uint32_t wg, uint32_t nwg) {
    const uint32_t tid = threadIdx.x, waves = blockDim.x / kWave;
    if constexpr (NG == 0) {
        const uint32_t wave = tid / kWave;
        float* wave_smem = smem + wave * gate_reduce_wave_words(p);
        for (uint32_t tile = wg + wave * nwg; tile < p.n_gate_tiles; tile += nwg * waves)   // spread over the workgroups first
            gate_reduce_tile_wide<T>(p, tile, wave_smem, int(tid % kWave));
    } else {
        constexpr int NL = (NG + 3) / 4;   // runs of 64 experts
        const uint32_t groups = waves / 4, group = tid / (4 * kWave), gtid = tid % (4 * kWave);
        uint32_t* gsm = reinterpret_cast<uint32_t*>(smem) + group * gate_group_words(p.E, p.k, p.is_training != 0);
        // tiles wg + j * nwg of the workgroup, j = 0 .. count-1; group g takes j = g, g + groups, ...
        const uint32_t count = wg < p.n_gate_tiles ? ceil_div_u32(p.n_gate_tiles - wg, nwg) : 0u;
        for (uint32_t j0 = 0; j0 < count; j0 += groups) {
            const uint32_t j = j0 + group;
            gate_reduce_group<T, NL>(p, wg + j * nwg, j < count, gsm, gtid);
        }
    }
}
// LDS words per wavefront of the reduce phase for more than 256 experts (a histogram and the picks)
__host__ __device__ inline uint32_t gate_reduce_wave_words(const LayerParams& p) { return p.E + kGateTileTokens * p.k; }
// LDS bytes of the reduce phase of a workgroup of `threads` threads
inline size_t gate_reduce_smem_bytes(const LayerParams& p, uint32_t threads) {
    if (p.E > 256) return size_t(threads / kWave) * gate_reduce_wave_words(p) * sizeof(float);
    return size_t(threads / (4 * kWave)) * gate_group_words(p.E, p.k, p.is_training != 0) * sizeof(float);
}

// ------------------------------------------------------------------------------------ phased
template <typename T>
__global__ __launch_bounds__(kGemmThreads, 1) void gate_gemm_kernel(const LayerParams p) {
    extern __shared__ __attribute__((aligned(16))) char gate_gemm_smem[];
    if constexpr (sizeof(T) == 2) gate_gemm_phase<T>(p, gate_gemm_smem, blockIdx.x, gridDim.x);
}
template <typename T, int NG>
__global__ __launch_bounds__(kPhaseThreads) void gate_reduce_kernel(const LayerParams p) {
    extern __shared__ __attribute__((aligned(16))) float gate_reduce_smem[];
    if constexpr (sizeof(T) == 2) gate_reduce_phase<T, NG>(p, gate_reduce_smem, blockIdx.x, gridDim.x);
}

// One gate unit per workgroup, with as many wavefronts as the persistent kernel's workgroups have:
// the split of the hidden dimension, and with it the summation order of the logits, is the same
// in both modes.
template <typename T, int NG>
__global__ __launch_bounds__(TileShape<T>::kThreads) void gate_kernel(const LayerParams p) {
    extern __shared__ __attribute__((aligned(16))) float gate_smem[];
    if constexpr (NG == 0) gate_unit_wide<T, TileShape<T>::kThreads / kWave>(p, blockIdx.x, gate_smem);
    else gate_unit<T, NG, TileShape<T>::kThreads / kWave>(p, blockIdx.x, gate_smem);
}

// One projection of every expert as a persistent grid with a static schedule: workgroup b takes
// the tiles b, b + G, b + 2G, ... of the list (expert, column block, row block). Consecutive
// workgroup ids land on consecutive XCDs, so with E a multiple of 8 expert e stays on XCD e % 8:
// all tiles that share its weights and its activation rows meet in one L2. Row blocks vary
// fastest so that the tiles re-reading one weight tile run together.
template <typename T, int V>
__global__ __launch_bounds__((TileShape<T, V>::kThreads), (TileShape<T, V>::kPerCu)) void expert_gemm_kernel(const LayerParams p, uint32_t kind,
                                                               uint32_t tiles_m, uint32_t tiles_n) {
    extern __shared__ __attribute__((aligned(16))) char gemm_smem[];
    uint32_t* s_task = reinterpret_cast<uint32_t*>(gemm_smem);
    const uint32_t per_expert = tiles_m * tiles_n, total = p.E * per_expert;
    uint32_t i = blockIdx.x;
    auto next = [&]() {
        Task t{};
        if (threadIdx.x == 0) {
            for (; i < total; i += gridDim.x) {
                uint32_t e, rem;
                if (p.E % kXcds == 0) {
                    const uint32_t xcd = i % kXcds, j = i / kXcds;
                    e = xcd + kXcds * (j / per_expert);
                    rem = j % per_expert;
                } else {
                    e = i / per_expert;
                    rem = i % per_expert;
                }
                const uint32_t mtile = rem % tiles_m;
                const uint32_t rows = kept_rows<false>(p, e);
                if (mtile * TileShape<T, V>::BM >= rows) continue;   // the expert has fewer rows
                t.e = e; t.rows = rows; t.kind = kind; t.mtile = mtile; t.ntile = rem / tiles_m; t.ready = 1; t.valid = 1;
                t.narrow = narrow_block<T, V>(rows, mtile);
                i += gridDim.x;
                break;
            }
        }
        return broadcast_task(s_task, t);
    };
    expert_loop<T, V>(p, gemm_smem + kPhasedGemmHeader, s_task, Readiness{nullptr, 0, 0, 0}, nullptr, next);
}

template <typename T>
__global__ __launch_bounds__(kPhaseThreads) void combine_kernel(const LayerParams p) {
    const uint32_t token = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p.is_training && blockIdx.x == gridDim.x - 1 && (threadIdx.x >> 6) == 3) gate_loss_finalize(p);
    combine_tokens<T>(p, token, p.S);
}

// ------------------------------------------------------------------------------------ fused
template <typename T, int NG, int V>
__global__ __launch_bounds__((TileShape<T, V>::kThreads), (TileShape<T, V>::kPerCu)) void fused_kernel(const LayerParams p, uint32_t seq,
                                                                      uint32_t mt_max, uint32_t dynamic_lag, uint32_t policy) {
    static_assert(sizeof(Segment) == 8, "segment table sizing");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int BM = TileShape<T, V>::BM, BN = TileShape<T, V>::BN;
    constexpr uint32_t kThreads = TileShape<T, V>::kThreads;
    constexpr uint32_t kWaves = kThreads / kWave;
    const uint32_t tid = threadIdx.x, wave = tid >> 6;
    const uint32_t nwg = gridDim.x;
    uint32_t* sched = p.sched;
    unsigned long long* stamp = p.stamps + size_t(blockIdx.x) * kStampWords;
    if (tid == 0) stamp[0] = wall_clock64();

    // The XCD this workgroup really runs on (hardware register XCC_ID): all tiles of an expert are
    // queued on one XCD, so that its weights, its gathered rows and the h1 rows handed from its
    // up-projection to its down-projection all live in one L2. Every workgroup also takes a rank
    // among the workgroups of its XCD, which the static schedule strides by.
    const uint32_t xcd = __builtin_amdgcn_s_getreg((3 << 11) | 20) & (kXcds - 1);
    uint32_t* const members_now = sched + kSchedMembers + (seq & 1u) * kXcds * kSchedLine;
    uint32_t my_rank = 0;
    if (tid == 0) my_rank = atomic_add_agent(members_now + xcd * kSchedLine, 1u);

    // ---- phase 0: gate. Workgroup 0 also resets this launch's tickets and readiness counters
    // (nothing reads them before the second barrier) and the next launch's member counts.
    if (blockIdx.x == 0) {
        // (written through the L2 like everything that crosses workgroups: the others hit these
        // words with device-scope atomics)
        if (tid < uint32_t(kXcds)) {
            atomic_store_relaxed(sched + kSchedTicket + tid * kSchedLine, 0u);
            atomic_store_relaxed(sched + kSchedMembers + (((seq + 1u) & 1u) * kXcds + tid) * kSchedLine, 0u);
        }
        for (uint32_t i = tid; i < p.E * mt_max; i += kThreads) atomic_store_relaxed(sched + kSchedReady + i, 0u);
    }
    bool gate_done = false;
    if constexpr (sizeof(T) == 2 && (NG == 0 || NG >= 8)) {   // more than 64 experts
        if (p.gate_splits) {
            // logits as a tiled product, then (behind a grid-wide barrier) one wavefront per 16-token tile
            gate_gemm_phase<T>(p, smem, blockIdx.x, nwg);
            grid_barrier(sched, p.wait_ticks, 3, seq, nwg);
            gate_reduce_phase<T, NG>(p, reinterpret_cast<float*>(smem), blockIdx.x, nwg);
            gate_done = true;
        }
    }
    if (!gate_done)
        for (uint32_t unit = blockIdx.x; unit < ceil_div_u32(p.n_gate_tiles, gate_unit_blocks<NG>()); unit += nwg) {
            if constexpr (NG == 0) gate_unit_wide<T, int(kWaves)>(p, unit, reinterpret_cast<float*>(smem));
            else gate_unit<T, NG, int(kWaves)>(p, unit, reinterpret_cast<float*>(smem));
        }
    if (tid == 0) stamp[1] = wall_clock64();
    grid_barrier(sched, p.wait_ticks, 0, seq, nwg);
    if (tid == 0) stamp[2] = wall_clock64();

    // LDS map of the expert phase: row blocks per expert | queue starts, totals, task | segments | GEMM tile
    uint32_t* s_rows = reinterpret_cast<uint32_t*>(smem);                       // [E] rows kept
    uint16_t* s_mt = reinterpret_cast<uint16_t*>(smem + 4 * lds_experts(p.E));  // [E] row blocks
    uint32_t* s_qseg = reinterpret_cast<uint32_t*>(smem + lds_queue_offset(p.E));   // [9] first segment of each queue
    uint32_t* s_qtot = s_qseg + 16;                                             // [8] tickets in each queue
    uint32_t* s_task = s_qtot + 8;                                              // [kTaskWords] task broadcast slot
    uint32_t* s_qup = s_task + kTaskWords;                                      // [8] up-projection tickets in each queue
    // static schedule: [1] rank of the workgroup among those of its XCD, [3] next ticket of the
    // workgroup, [5] every XCD holds the same number of workgroups. Thread 0's own words live here
    // rather than in registers that would stay occupied through the GEMM main loop.
    uint32_t* s_static = s_qup + 8;
    // [8] the ticket from which a queue hands out its last down-projection tiles as halves of 128
    // rows, two tickets per tile (~0: none)
    uint32_t* s_qhalf = s_static + 6;
    static_assert((16 + 8 + kTaskWords + 8 + 6 + 8) * 4 <= kLdsQueue, "queue header");
    Segment* s_seg = reinterpret_cast<Segment*>(smem + lds_queue_offset(p.E) + kLdsQueue);   // at most 2*E segments
    char* s_gemm = smem + fused_lds_header(p.E);
    const uint32_t tn_up = ceil_div_u32(p.I, BN), tn_down = ceil_div_u32(p.H, BN);

    // Which queue (XCD) an expert goes to. With more than 64 experts they are dealt out in descending
    // order of their rows, forwards and backwards in turn (queues 0..7, then 7..0, ...), so that every
    // queue holds about the same number of rows as well as of experts: an expert's tiles cost the more
    // the more rows it really holds (padding rows repeat one address). 256-expert top-8 shape: 2.92
    // against 2.96 ms per forward with the placement by index. Every workgroup computes the same
    // placement from the same counts.
    //   s_place[q * per_q + i]: the i-th expert of queue q.
    const uint32_t per_q = ceil_div_u32(p.E, kXcds);
    uint16_t* s_place = reinterpret_cast<uint16_t*>(s_gemm + size_t(kWaves) * p.E * sizeof(uint32_t));
    auto place = [&](uint32_t e) {
        const uint32_t mine = s_rows[e];
        uint32_t rank = 0;   // experts with more rows, or as many and a lower index
        // (sixteen counts per trip to LDS; the array is padded to a multiple of 64 words)
        for (uint32_t o0 = 0; o0 < p.E; o0 += 16) {
            u32x4 v[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) v[j] = *reinterpret_cast<const u32x4*>(s_rows + o0 + 4 * j);
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) {
                const uint32_t o = o0 + j, other = v[j / 4][j % 4];
                rank += uint32_t(o < p.E && (other > mine || (other == mine && o < e)));
            }
        }
        const uint32_t round = rank / kXcds, pos = rank % kXcds;
        s_place[((round & 1u) ? kXcds - 1 - pos : pos) * per_q + round] = uint16_t(e);
    };
    // Up to 64 experts keep the placement by index (expert e in queue e mod 8, nothing to look up):
    // with at most eight experts to a queue the ranking costs the slot phase more than even rows bring.
    const bool by_index = p.E <= uint32_t(kWave);
    auto expert_at = [&](uint32_t q, uint32_t i) -> uint32_t {
        if (by_index) return q + kXcds * i;
        return s_place[q * per_q + i];
    };
    // experts in queue q: the full rounds, and the last, partial one from whichever end it starts at
    // (always from queue 0 with the placement by index)
    auto experts_in = [&](uint32_t q) {
        const uint32_t full = p.E / kXcds, rest = p.E % kXcds;
        const bool backwards = !by_index && (full & 1u);
        return full + uint32_t(rest != 0 && (backwards ? q >= kXcds - rest : q < rest));
    };

    // ---- phase 1: slots in token order
    {
        // Rows and row blocks per expert and the workgroups per XCD, for the queues of the expert
        // phase: what this reads (the routed counts the gate accumulated, the member counts) has been
        // complete since the first barrier, so its trips to memory ride along with the slot tiles. The threads at the top of the workgroup take it:
        // the slot tiles go to the wavefronts at the bottom.
        if (tid == kThreads - 1) {
            // the static schedule needs every XCD to hold the same number of workgroups
            uint32_t seen[kXcds];   // all eight asked for before the first answer is looked at
            for (uint32_t j = 0; j < kXcds; ++j) seen[j] = atomic_load_relaxed(members_now + j * kSchedLine);
            bool even = nwg % kXcds == 0;
            for (uint32_t j = 0; j < kXcds; ++j) even = even && seen[j] == nwg / kXcds;
            s_static[5] = even;
        }
        for (uint32_t e = kThreads - 1 - tid; e < p.E; e += kThreads) {
            const uint32_t routed = routed_count(p, e);
            const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
            const uint32_t rows = routed < cap ? routed : cap;   // consumers clamp the routed count to the capacity (packet.cuh:85,112-113)
            s_rows[e] = rows;
            s_mt[e] = uint16_t(ceil_div_u32(rows, BM));
        }
        // (the slot tiles' scratch sits in the GEMM tile's memory, clear of the words above)
        uint32_t* base = reinterpret_cast<uint32_t*>(s_gemm) + wave * p.E;
        // wavefront w of workgroup b takes tile b + w * nwg: the tiles spread over all CUs
        for (uint32_t t0 = blockIdx.x; t0 < p.n_gate_tiles; t0 += nwg * kWaves)
            slot_tile(p, t0 + wave * nwg, t0 + wave * nwg < p.n_gate_tiles, base);
        if (!by_index) {
            __syncthreads();   // the counts of all wavefronts
            for (uint32_t e = tid; e < p.E; e += kThreads) place(e);
        }
        uint32_t* other = p.super_count + size_t((p.epoch & 1u) ^ 1u) * p.n_super * p.E;
        for (uint32_t i = blockIdx.x * kThreads + tid; i < p.n_super * p.E; i += nwg * kThreads) other[i] = 0u;
    }
    if (tid == 0) stamp[3] = wall_clock64();

    // ---- phase 2: expert tiles from the per-XCD queues (by ticket, or by stride in the static schedule)
    // The queues of the expert phase are set up while this workgroup waits for the others to finish
    // the slot phase: what the set-up reads (the rows per expert worked out above, the workgroups
    // per XCD) has been complete since the first barrier.
    const uint32_t members = nwg / kXcds;
    bool use_static = false;
    grid_barrier(sched, p.wait_ticks, 1, seq, nwg, [&] {
        __syncthreads();   // the rows per expert and their queues are in place
        // Static or dynamic schedule: every workgroup decides alike, from the same counters.
        // Static: each XCD's workgroups stride through their queue (all its up tiles, then all its
        // down tiles) by their rank: no tickets, no stealing, nothing written back from the L2 per
        // tile. It needs every XCD to hold the same number of workgroups, and it pays only when no
        // queue would keep its XCD busy for longer than freely handed-out tiles keep the grid busy.
        // Thread q sets up queue q; its segments start at a fixed place, two per expert of the queue.
        const uint32_t my_nq = tid < uint32_t(kXcds) ? experts_in(tid) : 0u;
        if (tid < uint32_t(kXcds)) {
            uint32_t blocks = 0;
            for (uint32_t i = 0; i < my_nq; ++i) blocks += s_mt[expert_at(tid, i)];
            s_qtot[tid] = blocks;
        }
        if (tid == 0) {
            s_static[1] = my_rank;
            s_static[3] = my_rank;
        }
        __syncthreads();
        {
            // rounds = tiles one workgroup works through in a projection. Strided, an XCD needs
            // ceil(its tiles / its workgroups); handed out freely, the grid needs at least
            // ceil(all tiles / all workgroups). Static loses nothing when no XCD needs more.
            uint32_t hi = 0, sum = 0;
            for (uint32_t q = 0; q < kXcds; ++q) {
                const uint32_t blocks = s_qtot[q];
                hi = blocks > hi ? blocks : hi;
                sum += blocks;
            }
            const uint32_t m = members ? members : 1u;
            const bool balanced = ceil_div_u32(hi * tn_up, m) <= ceil_div_u32(sum * tn_up, m * kXcds) &&
                                  ceil_div_u32(hi * tn_down, m) <= ceil_div_u32(sum * tn_down, m * kXcds);
            // the same in every lane: keep it in a scalar register
            use_static = __builtin_amdgcn_readfirstlane(int(s_static[5] != 0 && balanced_or_forced(policy, balanced))) != 0;
        }
        __syncthreads();   // the row-block sums above shared s_qtot with the ticket totals below
        if (tid < uint32_t(kXcds)) {
            const uint32_t q = tid, nq = my_nq;
            uint32_t first = 0;   // two segments per expert of the queues before this one
            for (uint32_t j = 0; j < q; ++j) first += 2 * experts_in(j);
            uint32_t nseg = first;
            s_qseg[q] = first;
            if (q == kXcds - 1) s_qseg[kXcds] = 2 * p.E;
            const uint32_t lag = use_static ? nq : dynamic_lag;   // static: all ups, then all downs
            uint32_t ticket = 0, ups = 0;
            // up-projection of expert i, then down-projection of expert i - lag: a down tile is
            // handed out only after `lag` further experts' worth of tickets, by which time the
            // up tiles it depends on have normally been stored.
            for (uint32_t i = 0; i < nq + lag; ++i) {
                if (i < nq) {
                    const uint32_t e = expert_at(q, i);
                    s_seg[nseg++] = Segment{uint16_t(e), 0, 0, ticket};
                    ticket += uint32_t(s_mt[e]) * tn_up;
                    ups += uint32_t(s_mt[e]) * tn_up;
                }
                if (i >= lag && i - lag < nq) {
                    const uint32_t e = expert_at(q, i - lag);
                    s_seg[nseg++] = Segment{uint16_t(e), 1, 0, ticket};
                    ticket += uint32_t(s_mt[e]) * tn_down;
                }
            }
            // Freely handed-out tiles end raggedly: the workgroups of an XCD run in step, so a last
            // round that is not full leaves the others idle for a whole tile, and a workgroup of
            // another XCD that takes one of the last tiles finishes a whole tile later. Where the
            // kernel holds both tile heights, the last down-projection tiles of a queue (half a round's
            // worth) are therefore handed out as two tickets of 128 rows each. What a tile computes
            // does not depend on its height (same instructions, same order along K).
            uint32_t halved = 0;
            if constexpr (kMixedHeights<T, V> && KLEOS_TUNE_HALVED_TAIL != 0) {
                if (!use_static && nq != 0 && lag != 0) {
                    const uint32_t last = uint32_t(s_mt[expert_at(q, nq - 1)]) * tn_down;   // the queue ends with this expert's down tiles
                    halved = last < members / 2 ? last : members / 2;
                }
            }
            s_qhalf[q] = halved ? ticket - halved : ~0u;
            s_qtot[q] = ticket + halved;
            s_qup[q] = ups;
        }
        __syncthreads();
    });
    if (tid == 0) { stamp[4] = wall_clock64(); stamp[14] = use_static; }

    uint32_t q_off = 0;   // queues already found empty, starting from this workgroup's own XCD
    uint32_t q_dead = 0;  // bit q: queue q was seen exhausted
    bool q_scanned = false;
    const Readiness rd{sched, mt_max, tn_up, p.wait_ticks};
    // Fills in the tile behind a ticket; false for a ticket that stands for no rows (the second
    // half of a halved row block that holds at most 128 rows).
    auto decode = [&](Task& t, uint32_t q, uint32_t ticket) -> bool {
        uint32_t half = 0, halved = 0;
        const uint32_t from = s_qhalf[q];
        if (ticket >= from) {   // two tickets per tile from here on
            half = (ticket - from) & 1u;
            halved = 1;
            ticket = from + (ticket - from) / 2;
        }
        uint32_t sg = s_qseg[q];
        const uint32_t sg_end = s_qseg[q + 1];
        while (sg + 1 < sg_end && s_seg[sg + 1].start <= ticket) ++sg;
        t.e = s_seg[sg].expert;
        t.kind = s_seg[sg].kind;
        const uint32_t local = ticket - s_seg[sg].start;
        t.mtile = local % s_mt[t.e];
        t.ntile = local / s_mt[t.e];
        t.rows = s_rows[t.e];
        t.narrow = narrow_block<T, V>(t.rows, t.mtile);
        if (half && t.narrow) return false;   // the first half held all its rows
        t.narrow |= halved;
        t.half = half;
        t.valid = 1;
        return true;
    };
    auto next = [&]() {
        Task t{};
        if (tid == 0 && use_static) {
            const uint32_t ticket = s_static[3];
            if (ticket < s_qtot[xcd]) {
                decode(t, xcd, ticket);   // (no halved tiles in the static schedule)
                t.dep = t.kind == 0 ? 0u : atomic_load_relaxed(rd.counter(t));
                t.ready = t.kind == 0 || rd.complete(t.dep);
                s_static[3] = ticket + members;
            }
        } else if (tid == 0) {
            while (q_off < kXcds) {
                const uint32_t q = (xcd + q_off) % kXcds;
                if (q_off != 0 && !q_scanned) {
                    // Leaving the own queue: read every ticket counter once, all loads in flight
                    // together, so that exhausted foreign queues (the normal case when the load is
                    // balanced) cost one round trip in total instead of one atomic each.
                    uint32_t seen[kXcds];
                    for (uint32_t j = 0; j < kXcds; ++j) seen[j] = atomic_load_relaxed(sched + kSchedTicket + j * kSchedLine);
                    for (uint32_t j = 0; j < kXcds; ++j) q_dead |= uint32_t(seen[j] >= s_qtot[j]) << j;
                    q_scanned = true;
                }
                if (s_qtot[q] == 0 || ((q_dead >> q) & 1u)) { ++q_off; continue; }
                const uint32_t ticket = atomic_add_agent(sched + kSchedTicket + q * kSchedLine, 1u);
                if (ticket >= s_qtot[q]) { ++q_off; continue; }
                if (!decode(t, q, ticket)) continue;
                t.foreign = q_off != 0;
                t.dep = t.kind == 0 ? 0u : atomic_load_relaxed(rd.counter(t));
                t.ready = t.kind == 0 || rd.complete(t.dep);
                break;
            }
        }
        return broadcast_task(s_task, t);
    };
    expert_loop<T, V>(p, s_gemm, s_task, rd, stamp + 8, next);
    if (tid == 0) stamp[5] = wall_clock64();
    grid_barrier(sched, p.wait_ticks, 2, seq, nwg);
    if (tid == 0) stamp[6] = wall_clock64();

    // ---- phase 3: combine, one token per wavefront
    if (p.is_training && blockIdx.x == nwg - 1 && wave == kWaves - 1) gate_loss_finalize(p);
    combine_tokens<T>(p, blockIdx.x * kWaves + wave, nwg * kWaves);
    __syncthreads();
    if (tid == 0) stamp[7] = wall_clock64();
}

template <typename T, int NG, int V>
size_t fused_smem_bytes(uint32_t E) {
    size_t need = fused_lds_header(E) + gemm_smem_bytes<T, V>();
    const size_t gate = gate_smem_floats<NG>(TileShape<T>::kThreads / kWave) * sizeof(float);
    // the slot tiles' scratch sits behind the header of the expert phase
    const size_t slots = fused_lds_header(E) + (TileShape<T>::kThreads / kWave) * size_t(E) * sizeof(uint32_t) +
                         kXcds * size_t(ceil_div_u32(E, kXcds)) * sizeof(uint16_t);   // and the experts of each queue behind it
    if (gate > need) need = gate;
    if (slots > need) need = slots;
    if constexpr (sizeof(T) == 2) {
        const size_t product = GateGemm<T>::kSmemBytes;
        // reduce phase: per wavefront a histogram and the picks (more than 256 experts), or per group
        // of four wavefronts the picks, a histogram and the probabilities of a tile (k <= E <= 256)
        const size_t reduce = E > 256 ? (TileShape<T>::kThreads / kWave) * size_t(E + kGateTileTokens * kWideGateMaxK) * sizeof(float)
                                      : (TileShape<T>::kThreads / (4 * kWave)) * size_t(gate_group_words(256, 256, true)) * sizeof(float);
        if (product > need) need = product;
        if (reduce > need) need = reduce;
    }
    return need;
}

inline int gate_groups(uint32_t E) {
    const uint32_t g = ceil_div_u32(E, 16);
    if (g <= 1) return 1;
    if (g <= 2) return 2;
    if (g <= 4) return 4;
    if (g <= 8) return 8;
    return 16;
}

// Calls f(integral_constant<int, V>) with the tile variant of the layer: the narrow tile when no
// expert can hold more than kNarrowRows rows (16-bit Elements only).
template <typename T, typename F>
hipError_t dispatch_variant(const LayerParams& p, F&& f) {
    if constexpr (sizeof(T) == 2) {
        const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
        if (cap <= kNarrowRows) return f(std::integral_constant<int, 1>{});
        if (cap >= kSharedRows) return f(std::integral_constant<int, 2>{});
    }
    return f(std::integral_constant<int, 0>{});
}

// Calls f(integral_constant<int, NG>) with the expert groups of the gate: 0 = the wide gate.
template <typename F>
hipError_t dispatch_groups(uint32_t E, F&& f) {
    if (E > 16 * kMaxGateGroups) return f(std::integral_constant<int, 0>{});
    switch (gate_groups(E)) {
        case 1: return f(std::integral_constant<int, 1>{});
        case 2: return f(std::integral_constant<int, 2>{});
        case 4: return f(std::integral_constant<int, 4>{});
        case 8: return f(std::integral_constant<int, 8>{});
        default: return f(std::integral_constant<int, 16>{});
    }
}

}  // namespace

// ------------------------------------------------------------------------------------ launchers per Element type
template <typename T>
hipError_t launch_gate_t(const LayerParams& p, int num_cus, hipStream_t s) {
    if (p.gate_splits) {
        return dispatch_groups(p.E, [&](auto ng) -> hipError_t {
            constexpr int NG = decltype(ng)::value;
            if constexpr (sizeof(T) == 2) {
                auto product = gate_gemm_kernel<T>;
                constexpr int smem = GateGemm<T>::kSmemBytes;
                static bool prepared = false;
                if (!prepared) {
                    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(product),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem);
                    if (err != hipSuccess) return err;
                    prepared = true;
                }
                uint32_t grid = gate_gemm_tiles(p);
                if (grid > uint32_t(num_cus)) grid = uint32_t(num_cus);
                hipLaunchKernelGGL(product, dim3(grid), dim3(kGemmThreads), smem, s, p);
                hipError_t err = hipGetLastError();
                if (err != hipSuccess) return err;
                // one tile per group of four wavefronts (per wavefront above 256 experts)
                const uint32_t reduce_grid = p.E > 256 ? ceil_div_u32(p.n_gate_tiles, kPhaseThreads / kWave) : p.n_gate_tiles;
                hipLaunchKernelGGL((gate_reduce_kernel<T, NG>), dim3(reduce_grid), dim3(kPhaseThreads),
                                   gate_reduce_smem_bytes(p, kPhaseThreads), s, p);
                return hipGetLastError();
            } else {
                return hipErrorInvalidValue;
            }
        });
    }
    return dispatch_groups(p.E, [&](auto ng) -> hipError_t {
        constexpr int NG = decltype(ng)::value;
        auto kernel = gate_kernel<T, NG>;
        constexpr int smem = gate_smem_floats<NG>(TileShape<T>::kThreads / kWave) * sizeof(float);
        static bool prepared = false;   // once per (Element type, group count)
        if (!prepared && smem > 48 * 1024) {
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (err != hipSuccess) return err;
        }
        prepared = true;
        hipLaunchKernelGGL(kernel, dim3(ceil_div_u32(p.n_gate_tiles, gate_unit_blocks<NG>())), dim3(TileShape<T>::kThreads),
                           smem, s, p);
        return hipGetLastError();
    });
}

template <typename T>
hipError_t launch_expert_gemm_t(const LayerParams& p, int kind, int num_cus, hipStream_t s) {
    const uint32_t N = kind == 0 ? p.I : p.H;
    return dispatch_variant<T>(p, [&](auto variant) -> hipError_t {
        constexpr int V = decltype(variant)::value;
        const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
        const uint32_t tiles_m = ceil_div_u32(cap, TileShape<T, V>::BM), tiles_n = ceil_div_u32(N, TileShape<T, V>::BN);
        const uint32_t total = p.E * tiles_m * tiles_n;
        auto kernel = expert_gemm_kernel<T, V>;
        constexpr int smem = kPhasedGemmHeader + gemm_smem_bytes<T, V>();
        static int resident = 0;   // workgroups per CU, found once per Element type and tile variant
        if (resident == 0) {
            // more than 64 KB of dynamic LDS has to be asked for explicitly
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (err != hipSuccess) return err;
            int occ = 0;
            err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, TileShape<T, V>::kThreads, smem);
            if (err != hipSuccess) return err;
            if (occ < 1) return hipErrorLaunchOutOfResources;
            resident = occ;
        }
        // persistent grid: as many workgroups as stay resident, a multiple of the XCD count
        uint32_t grid = uint32_t(num_cus) * uint32_t(resident);
        if (grid > total) grid = (total + kXcds - 1) / kXcds * kXcds;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(TileShape<T, V>::kThreads), smem, s, p, uint32_t(kind), tiles_m, tiles_n);
        return hipGetLastError();
    });
}

template <typename T>
hipError_t launch_combine_t(const LayerParams& p, hipStream_t s) {
    const uint32_t grid = ceil_div_u32(p.S, 4);
    hipLaunchKernelGGL((combine_kernel<T>), dim3(grid), dim3(kPhaseThreads), 0, s, p);
    return hipGetLastError();
}

template <typename T>
hipError_t plan_fused_t(const LayerParams& p, int num_cus, FusedPlan* plan) {
    return dispatch_groups(p.E, [&](auto ng) -> hipError_t {
        constexpr int NG = decltype(ng)::value;
        return dispatch_variant<T>(p, [&](auto variant) -> hipError_t {
            constexpr int V = decltype(variant)::value;
            auto kernel = fused_kernel<T, NG, V>;
            const size_t smem = fused_smem_bytes<T, NG, V>(p.E);
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
            if (err != hipSuccess) return err;
            int occ = 0;
            err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, TileShape<T, V>::kThreads, smem);
            if (err != hipSuccess) return err;
            if (occ < 1) return hipErrorLaunchOutOfResources;
            if (occ > 2) occ = 2;
            // every workgroup must be resident at once: the kernel holds grid-wide barriers. The grid is
            // what the occupancy query says fits an otherwise idle device.
            plan->nwg = uint32_t(num_cus) * uint32_t(occ);
            plan->smem = smem;
            const uint32_t cap = p.EC < p.cap_rows ? p.EC : p.cap_rows;
            plan->mt_max = ceil_div_u32(cap, TileShape<T, V>::BM);
            // tickets that separate an expert's up tiles from its down tiles: about one wave of
            // the resident workgroups of a queue
            const uint32_t tiles_per_expert = plan->mt_max * ceil_div_u32(p.I, TileShape<T, V>::BN);
            plan->lag = ceil_div_u32(ceil_div_u32(plan->nwg, kXcds), tiles_per_expert ? tiles_per_expert : 1u);
            if (plan->lag < 1) plan->lag = 1;
            plan->kernel = reinterpret_cast<const void*>(kernel);
            plan->threads = TileShape<T, V>::kThreads;
            return hipSuccess;
        });
    });
}

// The instantiations for one Element type (each in the translation unit of that type).
#define KLEOS_INSTANTIATE_ELEMENT(T)                                                                       \
    template hipError_t launch_gate_t<T>(const LayerParams&, int, hipStream_t);                            \
    template hipError_t launch_expert_gemm_t<T>(const LayerParams&, int, int, hipStream_t);                \
    template hipError_t launch_combine_t<T>(const LayerParams&, hipStream_t);                              \
    template hipError_t plan_fused_t<T>(const LayerParams&, int, FusedPlan*);
// ... and what keeps every other translation unit from instantiating them.
#define KLEOS_EXTERN_ELEMENT(T)                                                                            \
    extern template hipError_t launch_gate_t<T>(const LayerParams&, int, hipStream_t);                     \
    extern template hipError_t launch_expert_gemm_t<T>(const LayerParams&, int, int, hipStream_t);         \
    extern template hipError_t launch_combine_t<T>(const LayerParams&, hipStream_t);                       \
    extern template hipError_t plan_fused_t<T>(const LayerParams&, int, FusedPlan*);

}  // namespace kleos_amd
