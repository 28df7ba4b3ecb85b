// Expert projections: C[m, n] = act(sum_k A[m, k] * W[n, k] + bias[n]) on one output tile, with
// the rows of A optionally gathered through the slot->token table, so the dispatch of the
// reference (packet::dispatch row copy into a per-expert heap cell, csrc/include/kleos/os/
// packet.cuh:151-160) never materialises: the gather happens while the tile is staged into LDS.
//
// Replaces processor::fGET + BlockMM + FAA (csrc/include/kleos/os/processor/processor.cuh:358-489,
// gemm.cuh:22-107). Rounding points are the reference's: fp32 accumulate, fp32 bias add and
// activation, one round-to-nearest-even to Element on store (processor.cuh:475).
#pragma once
#include <type_traits>
#include "device_common.hpp"

namespace kleos_amd {

// ------------------------------------------------------------------------------------------------
// 16-bit Elements (bf16, fp16), matrix cores. WAVES_M x WAVES_N wavefronts over a BM x BN tile.
//
// K is walked in slices of BK through a ring of LDS stages that the wavefronts fill with direct
// global->LDS loads (global_load_lds_dwordx4: each lane names a 16-byte global source, the 64 lanes
// of the instruction land in 1 KB of consecutive LDS). They never occupy a vector register. Rows of
// A are gathered through the slot->token table by giving each lane its token's row address.
// Slice kt+STAGES-1 is requested during slice kt, into the stage slice kt-1 was read from, its loads
// placed one by one behind the matrix instructions of the slice's first quarters (a slice's matrix
// instructions run in four equal quarters: one K step each with 32x32x16, half a K step with 16x16x32).
// With two stages the loads can instead run two slices ahead (AHEAD2): slice kt+2 is requested
// into the stage of slice kt as soon as every wavefront has read its last fragments of slice kt (a
// second workgroup barrier per slice, placed before the last quarter, whose matrix instructions
// the loads then follow one by one), so the memory pipeline holds requests across the wait for
// slice kt+1 instead of running empty at every slice boundary.
//
// LDS layout of a stage: rows of BK*2 bytes, 16-byte chunk c of row r stored at chunk position
// c ^ swizzle(r). The LDS of gfx950 has 64 banks of 4 bytes and serves a 16-byte access of 16 lanes
// per clock; the swizzle (128-byte rows: ((r>>1)&7) ^ ((r&1)<<2), 64-byte rows: (r>>2)&3) makes any
// 16 consecutive rows read at one chunk index cover all 64 banks. Because the LDS destination of a
// direct load is fixed by the lane number, the swizzle is applied on the global side: the lane
// that lands on position p of row r fetches chunk p ^ swizzle(r).
//
// The weight rows feed the matrix core's row operand and the activation rows its column operand,
// i.e. the core computes C^T: a lane then owns 4 consecutive output columns of one output row.
//
// The tile computation is split into the pieces a persistent workgroup overlaps across tiles:
//   begin()    per-lane source addresses + the loads of the bias and of the first STAGES-1 slices
//   mainloop() all K slices
//   finish()   bias, activation, rounding, transposition through LDS, coalesced stores
// A workgroup calls finish() of a tile, then begin() of its next one: the stores enter the memory
// pipeline ahead of the next tile's loads (measured: 2 % faster than the other order, in which the
// stores queue behind a slice of loads and hold the wavefronts that issue them), and the stage ring
// keeps turning across tiles (finish() stages its output in the stage of the last slice, which
// every wavefront has left; begin() follows behind a workgroup barrier of the caller).
// ------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_ptr;

// One direct global->LDS load: every lane names 16 bytes of global memory, and the 64 lanes' bytes
// land in the 1 KB of LDS at `dst` (the same address in all lanes; the instruction takes it from M0)
// in lane order. Written as inline assembly, not as the compiler's builtin, on purpose: the compiler
// cannot see the `s_waitcnt vmcnt` this file places by hand, so it takes every direct load it knows
// of for pending for ever, and in front of any later LDS read whose address it cannot tell apart
// from the loads' destinations it waits for all of them (`vmcnt(0)`) - which empties the pipeline of
// loads that run one or two K slices ahead. Whether it could tell them apart turned out to depend on
// the surrounding code (the same main loop lost 11 % inside one kernel and nothing inside another).
// The ordering these loads need is all explicit here: a wait for the wavefront's own loads, then a
// workgroup barrier, before anybody reads a stage; a barrier behind everybody's last read before a
// stage is written again. Loads the compiler does not know of only make its own waits stricter.
// (M0 is a register the compiler sets up itself right in front of each instruction that reads it
// and keeps nothing in; it warns about any statement that names it)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// `lds`: the LDS address of the 1 KB, a value the compiler holds in a scalar register (lds_address()
// plus offsets that are the same in all lanes).
template <bool NON_TEMPORAL>
__device__ __forceinline__ void direct_load16(const void* src, uint32_t lds) {
    // (one wait state between the write of M0 and the load that reads it)
    if constexpr (NON_TEMPORAL)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds), "v"(src) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds), "v"(src) : "memory", "m0");
}
#pragma clang diagnostic pop
// The LDS address of a pointer into the workgroup's LDS, in a scalar register.
__device__ __forceinline__ uint32_t lds_address(const char* p) {
    return __builtin_amdgcn_readfirstlane(uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const char*)p)));
}
// The wavefront's index within the workgroup, in a scalar register.
__device__ __forceinline__ uint32_t wave_index() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

// A 16-bit Element seen only as storage: addresses are computed in units of it, values are
// interpreted by the Element type the tile is instantiated with.
typedef uint16_t elem16_t;

// What one output tile needs, in scalar form (identical in every lane).
struct GemmTileArgs {
    const elem16_t* a_base;        // A rows (gathered through a_row_index when it is not null)
    const int32_t* a_row_index;
    uint32_t a_rows;               // rows behind a_base: gathered indices are clamped below it
    const elem16_t* a_pad;         // K zeros that stand in for the rows past m_valid (null: they re-read the last valid row)
    const elem16_t* b_base;        // first of the tile's weight rows
    const elem16_t* bias;          // first of the tile's bias entries
    elem16_t* c_base;              // output element (row 0, column 0) of the tile
    uint32_t lda, ldb, ldc, K;
    uint32_t k_first;              // K slice the tile starts with (it wraps around); below K / BK
    uint32_t m_valid, n_valid;     // rows / columns of the tile that exist
    uint32_t act;                  // 0 relu, 1 erf-gelu, 2 identity
};

// Where a tile's results go.
struct TileOut {
    elem16_t* c_base;              // output element (row 0, column 0) of the tile
    uint32_t ldc, m_valid, n_valid, act;
};

// The lane's thread index as a value the optimiser cannot trace back to threadIdx: whatever a
// phase derives from it is computed when the phase starts and dies when it ends, instead of
// being shared with the main loop and kept (or spilled) across it.
__device__ __forceinline__ uint32_t local_tid() {
    uint32_t t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

// Epilogue of a WAVES_M x WAVES_N wavefront grid whose wavefronts each hold a WM x WN block of the
// C^T accumulators: acc[ni][mi][v] is output column n = wn*WN + ni*32 + 8*(v/4) + 4*(lane/32) + v%4
// of output row m = wm*WM + mi*32 + lane%32, i.e. a lane owns 4 consecutive columns of 16 rows per
// 32x32 block. Bias, activation and the rounding to Element happen in registers; the wavefront
// then transposes 32-row x 64-column panels through a private LDS region of 4 KB at
// stage_mem + wave * 4096 (rows of 128 bytes, 16-byte chunk c of row r at position
// c ^ ((r >> 1) & 7)) so that the global stores are 16 bytes per lane and cover whole 128-byte
// lines of the output rows. The bias comes from LDS (bias_mem: the tile's BN entries): the epilogue
// issues no global load, so nothing in it ever waits for the stores it has in flight.
constexpr int kEpiloguePanelRows = 32;
// The output rows are stored with the agent-scope (sc1) policy, which writes them through the L2
// instead of leaving dirty lines there: other workgroups read them later in the same launch, on
// any XCD, and nothing then has to write a whole L2 back before it may tell them so. It also pays
// by itself where a launch writes far more output than the L2 holds (256-expert top-8 shape: 3.03
// against 3.11 ms per forward); neutral on the other shapes measured.
// STREAM_OUT adds the non-temporal hint: the rows pass through the L2 without staying there. For
// layers of many small experts, whose intermediate and output rows are many times the L2 and are
// read long after they were written (256-expert top-8 shape: 2 865 against 2 950 us per forward with
// both outputs streamed, 2 913 with the intermediate rows alone, 2 953 with the output rows alone);
// where the rows are read back soon, from the L2 that took them, it costs (64-expert shape 293
// against 287 us, 16-expert shape 154 against 146 us).
template <typename E, int WM, int WN, int WAVES_N, int ACT, bool STREAM_OUT>
__device__ __forceinline__ void epilogue16_act(const TileOut& t, f32x16 (&acc)[WN / 32][WM / 32], char* stage_mem,
                                               const char* bias_mem) {
    typedef typename Elem16<E>::vec4 vec4;
    constexpr int TM = WM / 32, kPanelRows = kEpiloguePanelRows;
    const uint32_t tid = local_tid();
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int fr_row = lane & 31, fr_half = lane >> 5;
    char* stg = stage_mem + wave * (kPanelRows * 128);
    const char* bias_lane = bias_mem + (wn * WN + 4 * fr_half) * 2;
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) {
#pragma unroll
        for (int pn = 0; pn < WN / 64; ++pn) {
#pragma unroll
            for (int nl = 0; nl < 2; ++nl) {
                const int ni = pn * 2 + nl;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const vec4 b4 = *reinterpret_cast<const vec4*>(bias_lane + (ni * 32 + 8 * q) * 2);
                    vec4 o;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[j] = static_cast<E>(activate<ACT>(acc[ni][mi][4 * q + j] + float(b4[j])));
                    *reinterpret_cast<vec4*>(stg + fr_row * 128 + (((nl * 4 + q) ^ ((fr_row >> 1) & 7)) << 4) + fr_half * 8) = o;
                }
            }
            // the same wavefront wrote and reads the region: LDS operations of one wavefront
            // complete in order
#pragma unroll
            for (int it = 0; it < kPanelRows * 8 / kWave; ++it) {
                const int id = it * kWave + lane;
                const int r = id >> 3, c = id & 7;
                const u32x4 v = load16(stg + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
                const uint32_t m = wm * WM + mi * 32 + r, n = wn * WN + pn * 64 + c * 8;
                if (m < t.m_valid && n < t.n_valid) {
                    constexpr int kAgentScope = STREAM_OUT ? 16 + 2 : 16;   // sc1 (+ nt)
                    // (a tile's rows lie within 2 GiB of its first element: 256 rows of at most 2^22 bytes)
                    __builtin_amdgcn_raw_buffer_store_b128(v, coherent_rows(t.c_base), int((size_t(m) * t.ldc + n) * sizeof(E)), 0,
                                                           kAgentScope);
                }
            }
        }
    }
}
template <typename E, int WM, int WN, int WAVES_N, bool STREAM_OUT>
__device__ __forceinline__ void epilogue16(const TileOut& t, f32x16 (&acc)[WN / 32][WM / 32], char* stage_mem,
                                           const char* bias_mem) {
    if (t.act == 0) epilogue16_act<E, WM, WN, WAVES_N, 0, STREAM_OUT>(t, acc, stage_mem, bias_mem);
    else if (t.act == 1) epilogue16_act<E, WM, WN, WAVES_N, 1, STREAM_OUT>(t, acc, stage_mem, bias_mem);
    else epilogue16_act<E, WM, WN, WAVES_N, 2, STREAM_OUT>(t, acc, stage_mem, bias_mem);
}

// The same epilogue for accumulators of 16 x 16 matrix-core tiles: acc[ni][mi][v] is output column
// n = wn*WN + ni*16 + 4*(lane/16) + v of output row m = wm*WM + mi*16 + lane%16 - again 4 consecutive
// columns per lane and tile, so the panels, their LDS layout and the stores are the ones above.
template <typename E, int WM, int WN, int WAVES_N, int ACT, bool STREAM_OUT>
__device__ __forceinline__ void epilogue16_act(const TileOut& t, f32x4 (&acc)[WN / 16][WM / 16], char* stage_mem,
                                               const char* bias_mem) {
    typedef typename Elem16<E>::vec4 vec4;
    constexpr int kPanelRows = kEpiloguePanelRows;
    const uint32_t tid = local_tid();
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int fr_row = lane & 15, fr_part = lane >> 4;
    char* stg = stage_mem + wave * (kPanelRows * 128);
    const char* bias_lane = bias_mem + (wn * WN + 4 * fr_part) * 2;
#pragma unroll
    for (int pm = 0; pm < WM / 32; ++pm) {
#pragma unroll
        for (int pn = 0; pn < WN / 64; ++pn) {
#pragma unroll
            for (int ml = 0; ml < 2; ++ml) {
                const int r = ml * 16 + fr_row;   // row of the panel
#pragma unroll
                for (int nl = 0; nl < 4; ++nl) {
                    const int ni = pn * 4 + nl;
                    const vec4 b4 = *reinterpret_cast<const vec4*>(bias_lane + ni * 16 * 2);
                    vec4 o;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[j] = static_cast<E>(activate<ACT>(acc[ni][pm * 2 + ml][j] + float(b4[j])));
                    // columns nl*16 + 4*fr_part .. + 3 of the panel: chunk 2*nl + fr_part/2, half fr_part%2
                    *reinterpret_cast<vec4*>(stg + r * 128 + (((2 * nl + (fr_part >> 1)) ^ ((r >> 1) & 7)) << 4) + (fr_part & 1) * 8) = o;
                }
            }
#pragma unroll
            for (int it = 0; it < kPanelRows * 8 / kWave; ++it) {
                const int id = it * kWave + lane;
                const int r = id >> 3, c = id & 7;
                const u32x4 v = load16(stg + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
                const uint32_t m = wm * WM + pm * 32 + r, n = wn * WN + pn * 64 + c * 8;
                if (m < t.m_valid && n < t.n_valid) {
                    constexpr int kAgentScope = STREAM_OUT ? 16 + 2 : 16;   // sc1 (+ nt)
                    __builtin_amdgcn_raw_buffer_store_b128(v, coherent_rows(t.c_base), int((size_t(m) * t.ldc + n) * sizeof(E)), 0,
                                                           kAgentScope);
                }
            }
        }
    }
}
template <typename E, int WM, int WN, int WAVES_N, bool STREAM_OUT>
__device__ __forceinline__ void epilogue16(const TileOut& t, f32x4 (&acc)[WN / 16][WM / 16], char* stage_mem,
                                           const char* bias_mem) {
    if (t.act == 0) epilogue16_act<E, WM, WN, WAVES_N, 0, STREAM_OUT>(t, acc, stage_mem, bias_mem);
    else if (t.act == 1) epilogue16_act<E, WM, WN, WAVES_N, 1, STREAM_OUT>(t, acc, stage_mem, bias_mem);
    else epilogue16_act<E, WM, WN, WAVES_N, 2, STREAM_OUT>(t, acc, stage_mem, bias_mem);
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in this order.
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// STREAM_B: the weight rows are loaded with the non-temporal cache policy: read once (or by a
// neighbour at the same moment), they pass through the L2 without displacing the activation rows
// that are shared (7.0 against 6.4 TB/s on a read-only stream of this shape).
// AHEAD2 (two stages only): the loads run two slices ahead, at the price of a second workgroup
// barrier per slice. It pays where the weights stream from HBM and a slice's loads take longer than
// its matrix work (headline shape: 301 against 315 us for the expert phase); where the matrix work
// dominates it needs SPREAD to pay (8-expert shape with hidden size 4096, both projections: 4.18 ms
// with all loads of a slice at once against 4.11 one slice ahead, 3.95 with them shared out 4 + 4).
// SPREAD (with AHEAD2): when the loads of a slice are issued. 0: all of them behind the matrix
// instructions of the last quarter of the slice two before it, which frees their stage. Otherwise
// only the first of them go there and the rest behind the first quarters of the next slice
// (spread_count: 1 = 4 + 4, 2 = 3 + 3 + 2 of the 8 loads of a wavefront). The CU's load path takes in
// about one 1 KB load every 36 clocks while all CUs stream; the 64 loads of a slice issued by eight
// wavefronts inside one K step queue up in front of it, and each wavefront's matrix instructions sit
// behind its loads in program order. Shared out evenly over all four K steps the last loads leave too
// late (4.07 ms at the shape above); one barrier per slice instead of two (the barrier in front of the
// last K step also standing for "the next slice has landed", its first fragments read behind that K
// step's matrix instructions) loses the lead time it needs: 3.98 ms.
#ifndef KLEOS_GEMM_BLOCK_SKIP
#define KLEOS_GEMM_BLOCK_SKIP 1
#endif
// MI: the matrix-core tile. 32: 32x32x16 instructions (16 values of K each, 16 accumulator registers);
// 16: 16x16x32 instructions (32 values of K, 4 accumulator registers). The smaller tile reads and
// writes half as many accumulator registers per multiply-add and draws less power for the same work
// (instruction loops on random bf16 operands held in registers, whole device: 2.08 against 1.84
// PFLOP/s at the same 1.31 kW), which is what bounds these kernels.
// RELEASE (with AHEAD2 and 16-row matrix tiles, whose slices have two K steps): where the barrier
// that frees a slice's stage sits. The fragments of the second K step are read behind the matrix
// instructions of the first, so a wavefront has finished with the stage half a slice before it
// finishes the slice. 0: the barrier stays in front of the last quarter. 2: it moves into the third
// quarter, kReleaseAt matrix instructions in (the last reads have returned by then), and the first
// loads of the slice after the next follow it there: a quarter of a slice more for them to land
// (8-expert shape with hidden size 4096: 3 088 against 3 115 us per forward; no difference at the
// 64- and 16-expert shapes). 1: all loads of that slice go behind the early barrier, half in the third
// and half in the last quarter, none into the next slice: every load has between one and one and a
// half slices to land (16-expert shape 146 against 150 us, 64-expert shape 284 against 287 us; the
// 8-expert shape loses, 3 177 against 3 115 us: its loads, bunched into half a slice, hold up the
// matrix instructions behind them).
// STREAM_OUT: the output rows are stored with the non-temporal hint (see the epilogue above).
template <typename E, int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES, bool STREAM_B, bool AHEAD2, int SPREAD = 0, int MI = 32,
          int RELEASE = 0, bool STREAM_OUT = false>
struct Gemm16 {
    typedef typename Elem16<E>::vec8 vec8;
    typedef typename Elem16<E>::vec4 vec4;
    static constexpr int kWaves = WAVES_M * WAVES_N;
    static constexpr int kThreads = kWaves * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;     // wavefront tile
    static constexpr int TM = WM / MI, TN = WN / MI;               // matrix-core tiles per wavefront
    static constexpr int KI = MI == 32 ? 16 : 32;                  // values of K one matrix instruction consumes
    static constexpr int kRowBytes = BK * 2;
    static constexpr int kRowsPerLoad = 1024 / kRowBytes;          // rows one direct load covers
    static constexpr int kChunks = kRowBytes / 16;                 // 16-byte chunks per row
    static constexpr int kABytes = BM * kRowBytes, kBBytes = BN * kRowBytes;
    static constexpr int kStage = kABytes + kBBytes;
    static constexpr int kBiasBytes = BN * 2;                      // one tile's bias entries
    static constexpr int kBiasOffset = STAGES * kStage;            // two bias slots behind the stage ring
    static constexpr int kSmemBytes = STAGES * kStage + 2 * kBiasBytes;
    static constexpr int LA = BM / (kRowsPerLoad * kWaves), LB = BN / (kRowsPerLoad * kWaves);
    static constexpr int kLoadsPerSlice = LA + LB;                 // per wavefront
    static constexpr int kSliceK = BK;                             // values of K per slice
    static constexpr int kSteps = BK / KI;                         // K steps per slice
    // 16-row tiles, wavefront tiles of four of them in height: a wavefront leaves out the blocks of 16
    // rows that hold no rows of the tile (64-expert shape with skewed routing: the experts' 13 039 rows
    // take the matrix instructions of 13 424 rows that way, of 14 656 with whole wavefronts left out only)
    static constexpr bool kBlockSkip = KLEOS_GEMM_BLOCK_SKIP != 0 && MI == 16 && TM == 4;
    static constexpr bool kEarlyRelease = RELEASE == 1;   // every load of a slice behind the early barrier of the slice two before it
    static constexpr int kReleaseAt = 4;                  // matrix instructions of the third quarter in front of the early barrier
    static_assert(RELEASE >= 0 && RELEASE <= 2);
    static_assert(RELEASE == 0 || (AHEAD2 && MI == 16 && kSteps == 2));
    static constexpr int kQuarters = 4;                            // a slice's matrix instructions in four equal runs
    static constexpr int kPerQuarter = TN * TM * kSteps / kQuarters;
    static constexpr int kPanelRows = kEpiloguePanelRows;          // epilogue staging: 32 rows x 64 columns per wavefront
    // loads of a slice (per wavefront) issued at the last quarter of the slice two before it [0] and at
    // quarters 0, 1, 2 of the slice before it [1..3]
    static constexpr int spread_count(int i) {
        constexpr int L = LA + LB;
        switch (SPREAD) {
            case 1: return i < 2 ? L / 2 : 0;                                                       // 4 4 0 0
            case 2: return i == 0 || i == 1 ? (3 * L) / 8 : (i == 2 ? L - 2 * ((3 * L) / 8) : 0);   // 3 3 2 0
            default: return i == 0 ? L : 0;                                                         // all at once
        }
    }
    static constexpr bool kEarlyFirst = RELEASE == 2;     // only the first loads move with the barrier; the others stay in the next slice
    static_assert(RELEASE != 2 || spread_count(3) == 0, "the third quarter carries no loads of the next slice");
    static_assert(SPREAD >= 0 && SPREAD <= 2);
    static_assert(SPREAD == 0 || (AHEAD2 && (LA + LB) % 8 == 0));
    static_assert(spread_count(0) + spread_count(1) + spread_count(2) + spread_count(3) == LA + LB);
    static_assert(BK == 32 || BK == 64);
    static_assert(MI == 32 || MI == 16);
    static_assert(kQuarters % kSteps == 0 && (TN * TM * kSteps) % kQuarters == 0);
    static_assert(!AHEAD2 || STAGES == 2);
    static_assert(STAGES >= 2 && STAGES <= 4);
    static_assert(WM % 32 == 0 && WN % 64 == 0);
    static_assert(BM % (kRowsPerLoad * kWaves) == 0 && BN % (kRowsPerLoad * kWaves) == 0);
    static_assert(kWaves * kPanelRows * 128 <= kStage, "epilogue staging must fit one stage");
    static_assert((STAGES - 1) * kLoadsPerSlice < 64);
    static_assert(kBiasBytes <= 1024, "one direct load brings the bias");

    static __device__ __forceinline__ int swizzle(int r) {
        if constexpr (BK == 64) return ((r >> 1) & 7) ^ ((r & 1) << 2);
        else return (r >> 2) & 3;
    }

    struct Tile {
        const elem16_t* pa[LA];
        const elem16_t* pb[LB];
        elem16_t* c_base;
        uint32_t ldc, m_valid, n_valid, k_tiles, act;
        uint32_t k_first;           // the kt-th slice the tile works on is slice (k_first + kt) % k_tiles of K
        int stage0;                 // stage of the tile's first slice; its kt-th slice uses (stage0 + kt) % STAGES
        int bias_slot;              // which of the two LDS bias slots holds this tile's bias
    };

    typedef std::conditional_t<MI == 32, f32x16, f32x4> AccTile;
    typedef AccTile Acc[TN][TM];

    static __device__ __forceinline__ int stage_of(const Tile& t, uint32_t kt) { return (t.stage0 + kt) % STAGES; }

    // the direct loads that bring K slice kt of the tile into its stage: activation rows first (they
    // come from L2 and return early), then the weight rows
    static __device__ __forceinline__ void issue_slice(const Tile& t, char* smem, uint32_t kt) {
        const uint32_t sa = lds_address(smem) + stage_of(t, kt) * kStage + 1024 * wave_index();   // this wavefront's first KB of the stage
        const uint32_t sb = sa + kABytes;
        uint32_t slice = kt + t.k_first;
        slice = slice >= t.k_tiles ? slice - t.k_tiles : slice;
        const uint32_t k0 = slice * BK;
#pragma unroll
        for (int i = 0; i < LA; ++i)
            direct_load16<false>(t.pa[i] + k0, sa + 1024 * kWaves * i);
#pragma unroll
        for (int i = 0; i < LB; ++i)
            direct_load16<STREAM_B>(t.pb[i] + k0, sb + 1024 * kWaves * i);
    }

    // Load number j (0 <= j < LA + LB) of a K slice: activation rows first (they come from L2 and return
    // early), then the weight rows.
    // (sa, sb: the LDS addresses of this wavefront's first KB of the stage's activation and weight rows)
    static __device__ __forceinline__ void issue_one(const Tile& t, uint32_t sa, uint32_t sb, uint32_t k0, int j) {
        if (j >= LA)
            direct_load16<STREAM_B>(t.pb[j - LA] + k0, sb + 1024 * kWaves * (j - LA));
        else
            direct_load16<false>(t.pa[j] + k0, sa + 1024 * kWaves * j);
    }
    // Loads first .. first + count - 1 of K slice kt.
    template <int FIRST, int COUNT>
    static __device__ __forceinline__ void issue_range(const Tile& t, char* smem, uint32_t kt) {
        const uint32_t sa = lds_address(smem) + stage_of(t, kt) * kStage + 1024 * wave_index();
        const uint32_t sb = sa + kABytes;
        uint32_t slice = kt + t.k_first;
        slice = slice >= t.k_tiles ? slice - t.k_tiles : slice;
        const uint32_t k0 = slice * BK;
#pragma unroll
        for (int j = 0; j < COUNT; ++j) issue_one(t, sa, sb, k0, FIRST + j);
    }

    // Per-lane source addresses, the load of the bias into LDS slot `bias_slot`, then the loads of
    // the first STAGES-1 slices. Activation rows past the valid range read zeros (a_pad; the last valid
    // row without it) and weight rows past it re-read the last valid row: their products land in
    // accumulator rows / columns that are never stored, and a matrix core that multiplies zeros draws
    // less power than one that multiplies data. The stages stage0 ..
    // stage0+STAGES-2 and the bias slot must not be in use by any wavefront. The bias load is the
    // oldest of the tile's loads, so the first wait of mainloop() covers it.
    static __device__ __forceinline__ void begin(Tile& t, const GemmTileArgs& g, int stage0, int bias_slot, char* smem) {
        const uint32_t tid = local_tid();
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int ld_r = lane / kChunks, ld_p = lane % kChunks;
        if (wave == 0 && lane < kBiasBytes / 16) {
            const uint32_t n = uint32_t(lane) * 8 < g.n_valid ? uint32_t(lane) * 8 : 0u;
            direct_load16<false>(g.bias + n, lds_address(smem) + kBiasOffset + bias_slot * kBiasBytes);
        }
        // The lane's source rows. The slot->token table was written earlier in the same launch,
        // possibly on another XCD: device-coherent loads, all in flight together (an index is clamped
        // to the table it points into, so that no value it could ever hold turns into an address
        // outside the caller's buffer).
        uint32_t src[LA];
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            const int row = kRowsPerLoad * (wave + kWaves * i) + ld_r;
            src[i] = row < int(g.m_valid) ? row : g.m_valid - 1;
        }
        if (g.a_row_index) {
#pragma unroll
            for (int i = 0; i < LA; ++i) src[i] = uint32_t(load_coherent(g.a_row_index + src[i]));
#pragma unroll
            for (int i = 0; i < LA; ++i) src[i] = src[i] < g.a_rows ? src[i] : g.a_rows - 1;
        }
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            const int row = kRowsPerLoad * (wave + kWaves * i) + ld_r;
            const elem16_t* from = g.a_base + size_t(src[i]) * g.lda;
            if (g.a_pad && row >= int(g.m_valid)) from = g.a_pad;
            t.pa[i] = from + ((ld_p ^ swizzle(row)) << 3);
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            const int row = kRowsPerLoad * (wave + kWaves * i) + ld_r;
            const uint32_t r = row < int(g.n_valid) ? row : g.n_valid - 1;
            t.pb[i] = g.b_base + size_t(r) * g.ldb + ((ld_p ^ swizzle(row)) << 3);
        }
        t.c_base = g.c_base; t.ldc = g.ldc;
        t.m_valid = g.m_valid; t.n_valid = g.n_valid; t.k_tiles = g.K / BK;
        t.k_first = g.k_first < t.k_tiles ? g.k_first : 0u;
        t.act = g.act; t.stage0 = stage0; t.bias_slot = bias_slot;
#pragma unroll
        for (int st = 0; st < STAGES - 1; ++st)
            if (uint32_t(st) < t.k_tiles) issue_slice(t, smem, st);
    }

    // `after_first_barrier()` is called by every thread once, right behind the workgroup barrier that
    // follows the wait for the tile's first slice. Every vector-memory operation a wavefront issued
    // before begin() of this tile has completed by then, in every wavefront: what a persistent
    // workgroup stored in the epilogue of its previous tile may be announced to other workgroups from
    // there without a wait of its own. (begin() must follow the previous tile's finish().)
    static __device__ __forceinline__ void mainloop(const Tile& t, Acc& acc, char* smem) {
        mainloop(t, acc, smem, [] {});
    }
    template <typename Hook>
    static __device__ __forceinline__ void mainloop(const Tile& t, Acc& acc, char* smem, Hook&& after_first_barrier) {
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        const int wm = wave / WAVES_N, wn = wave % WAVES_N;
        // a lane's share of an operand fragment: 16 bytes of row fr_row, the fr_part-th 8 values of the K step
        const int fr_row = lane & (MI - 1), fr_part = lane / MI;
        if (rows_absent(t, __builtin_amdgcn_readfirstlane(wave) / WAVES_N)) {   // (a scalar condition: the branch holds barriers)
            // None of this wavefront's rows exist (an expert with few rows): it brings its share of
            // every slice into LDS at the same points of the same sequence of barriers as the others,
            // and leaves the fragment reads and the matrix instructions out.
            if constexpr (kEarlyRelease) {
                constexpr int L = LA + LB;
                asm volatile("s_barrier" ::: "memory");
                if (t.k_tiles > 1) issue_range<0, L>(t, smem, 1);
                for (uint32_t kt = 0; kt < t.k_tiles; ++kt) {
                    if (kt + 1 < t.k_tiles) wait_vmcnt<L>();
                    else wait_vmcnt<0>();
                    asm volatile("s_barrier" ::: "memory");
                    if (kt == 0) after_first_barrier();
                    if (kt + 2 < t.k_tiles) {
                        asm volatile("s_barrier" ::: "memory");
                        issue_range<0, L>(t, smem, kt + 2);
                    }
                }
            } else if constexpr (AHEAD2) {
                constexpr int N0 = spread_count(0);
                asm volatile("s_barrier" ::: "memory");
                if (t.k_tiles > 1) issue_range<0, N0>(t, smem, 1);
                for (uint32_t kt = 0; kt < t.k_tiles; ++kt) {
                    if (kt + 1 < t.k_tiles) wait_vmcnt<N0>();
                    else wait_vmcnt<0>();
                    asm volatile("s_barrier" ::: "memory");
                    if (kt == 0) after_first_barrier();
                    if (kt + 1 < t.k_tiles) issue_range<N0, LA + LB - N0>(t, smem, kt + 1);
                    if (kt + 2 < t.k_tiles) {
                        asm volatile("s_barrier" ::: "memory");
                        issue_range<0, N0>(t, smem, kt + 2);
                    }
                }
            } else {
                for (uint32_t kt = 0; kt < t.k_tiles; ++kt) {
                    const uint32_t later = t.k_tiles - 1 - kt;
                    if (STAGES >= 4 && later >= 2) wait_vmcnt<(STAGES >= 4 ? 2 : 0) * kLoadsPerSlice>();
                    else if (STAGES >= 3 && later >= 1) wait_vmcnt<kLoadsPerSlice>();
                    else wait_vmcnt<0>();
                    asm volatile("s_barrier" ::: "memory");
                    if (kt == 0) after_first_barrier();
                    if (kt + (STAGES - 1) < t.k_tiles) issue_slice(t, smem, kt + STAGES - 1);
                }
            }
            return;
        }
#pragma unroll
        for (int ni = 0; ni < TN; ++ni)
#pragma unroll
            for (int mi = 0; mi < TM; ++mi)
#pragma unroll
                for (int v = 0; v < int(sizeof(AccTile) / sizeof(float)); ++v) acc[ni][mi][v] = 0.f;
        // Fragment addresses inside a stage. Rows MI apart share their swizzle, and K step ks only
        // flips the upper bits of the chunk position (a step spans 2 chunks of 16 bytes with the
        // 32-row tiles, 4 with the 16-row tiles), so one base per operand is enough: the address of
        // block i at step ks is (base ^ (ks << kStepShift)) + i * MI rows.
        constexpr int kStepShift = MI == 32 ? 5 : 6;
        const int rx = wm * WM + fr_row, rw = wn * WN + fr_row;
        const int base_x = rx * kRowBytes + ((fr_part ^ swizzle(rx)) << 4);
        const int base_w = kABytes + rw * kRowBytes + ((fr_part ^ swizzle(rw)) << 4);
        // The operand fragments of K step ks+1 are read from LDS while the matrix core works on step ks.
        // 32-row tiles: two sets of fragments, fw[ks & 1] and fx[ks & 1]. 16-row tiles have twice as many
        // fragments per step: the larger set (the `outer` one: x with tall wavefront tiles, w with wide
        // ones) is walked in the outer loop of a step, each of its fragments serving NI instructions in
        // a row and making way for its successor of the next step right behind them (one set of
        // registers, fo); only the smaller set is kept twice (fi[ks & 1]).
        constexpr bool kOuterX = TM >= TN;
        constexpr int NO = kOuterX ? TM : TN, NI = kOuterX ? TN : TM;
        static_assert(MI == 32 || (NI >= 2 && NO >= NI));
        // XB: how many of the wavefront's TM blocks of MI rows hold rows of the tile. The blocks behind
        // them are left out of the fragment reads and the matrix instructions (with the 16-row tiles, in
        // the configurations that take the trouble: kBlockSkip); their accumulators are never stored.
        auto body = [&](auto xb_tag) {
            constexpr int XB = decltype(xb_tag)::value;
            auto x_block_used = [](int mi) { return mi < XB; };
            vec8 fw[2][MI == 32 ? TN : 1], fx[2][MI == 32 ? TM : 1];
            vec8 fo[MI == 16 ? NO : 1], fi[2][MI == 16 ? NI : 1];
            const int base_o = kOuterX ? base_x : base_w, base_i = kOuterX ? base_w : base_x;
            auto read_fragments = [&](const char* st, int ks) {
                if constexpr (MI == 32) {
#pragma unroll
                    for (int ni = 0; ni < TN; ++ni) fw[ks & 1][ni] = __builtin_bit_cast(vec8, load16(st + (base_w ^ (ks << kStepShift)) + ni * MI * kRowBytes));
#pragma unroll
                    for (int mi = 0; mi < TM; ++mi) fx[ks & 1][mi] = __builtin_bit_cast(vec8, load16(st + (base_x ^ (ks << kStepShift)) + mi * MI * kRowBytes));
                } else {
#pragma unroll
                    for (int k = 0; k < NI; ++k)
                        if (kOuterX || x_block_used(k)) fi[ks & 1][k] = __builtin_bit_cast(vec8, load16(st + (base_i ^ (ks << kStepShift)) + k * MI * kRowBytes));
#pragma unroll
                    for (int o = 0; o < NO; ++o)
                        if (!kOuterX || x_block_used(o)) fo[o] = __builtin_bit_cast(vec8, load16(st + (base_o ^ (ks << kStepShift)) + o * MI * kRowBytes));
                }
            };
            // Where one load of slice kn comes from and goes to (load li < LA: activation rows, else weight rows).
            struct SliceLoads { uint32_t sa, sb, k0; };
            const uint32_t lds_wave = lds_address(smem) + 1024 * wave_index();
            auto loads_of = [&](uint32_t kn) {
                SliceLoads l;
                l.sa = lds_wave + stage_of(t, kn) * kStage;
                l.sb = l.sa + kABytes;
                uint32_t slice = kn + t.k_first;
                slice = slice >= t.k_tiles ? slice - t.k_tiles : slice;
                l.k0 = slice * BK;
                return l;
            };
            // A quarter of a slice's matrix instructions (one K step with the 32-row tiles, half a K step
            // with the 16-row tiles) in a pinned order: one matrix instruction, behind it one LDS read of the
            // next K step's fragments (behind the first TN + TM instructions of a step) and, with LOADS, one
            // global load of a later slice, and again. Issued as blocks - all reads, then all
            // matrix instructions - the two wavefronts of a SIMD took turns instead of overlapping, and a
            // slice's loads in a block in front of a K step held the matrix cores up (8 experts x 2560
            // rows, hidden size 4096, both projections: 3.80 ms in blocks, 3.49 with the reads interleaved,
            // 3.47 with the loads interleaved too; with operands resident in L2 3.49, 2.96 and 2.72).
            // The loads are a compile-time switch: a branch around matrix instructions makes the compiler keep
            // two copies of the accumulators.
            // `first_tag`, `count_tag`: the quarter carries the loads first .. first + count - 1 of the slice `l`
            // describes, evenly spaced behind its matrix instructions (count 0: none).
            // `sync_tag` (S >= 0): in front of the quarter's S-th matrix instruction the wavefront waits for its LDS
            // reads and for the workgroup; the quarter's loads come behind that point.
            auto quarter = [&](const char* st, auto q_tag, const SliceLoads& l, auto first_tag, auto count_tag, auto sync_tag) {
                constexpr int Q = decltype(q_tag)::value, FIRST = decltype(first_tag)::value, COUNT = decltype(count_tag)::value;
                constexpr int S = decltype(sync_tag)::value, J0 = S > 0 ? S : 0;
                constexpr int kParts = kQuarters / kSteps;                 // quarters per K step
                constexpr int ks = Q / kParts, part = Q % kParts;
                static_assert(COUNT <= kPerQuarter - J0);
                constexpr int kEvery = (kPerQuarter - J0) / (COUNT > 0 ? COUNT : 1);
#pragma unroll
                for (int j = 0; j < kPerQuarter; ++j) {
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (S >= 0) {
                        if (j == S) {
                            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
                            asm volatile("s_barrier" ::: "memory");
                        }
                    }
                    const int i = part * kPerQuarter + j;                  // the step's i-th matrix instruction
                    if constexpr (MI == 32) {
                        const int ni = i / TM, mi = i % TM;
                        acc[ni][mi] = Elem16<E>::mfma32(fw[ks & 1][ni], fx[ks & 1][mi], acc[ni][mi]);
                        if (ks + 1 < kSteps) {
                            const int nb = (ks + 1) & 1;
                            if (i < TN) fw[nb][i] = __builtin_bit_cast(vec8, load16(st + (base_w ^ ((ks + 1) << kStepShift)) + i * MI * kRowBytes));
                            else if (i < TN + TM) fx[nb][i - TN] = __builtin_bit_cast(vec8, load16(st + (base_x ^ ((ks + 1) << kStepShift)) + (i - TN) * MI * kRowBytes));
                        }
                    } else {
                        const int o = i / NI, k = i % NI;
                        if (x_block_used(kOuterX ? o : k)) {   // (folds at compile time: o and k are unrolled)
                            if constexpr (kOuterX) acc[k][o] = Elem16<E>::mfma16(fi[ks & 1][k], fo[o], acc[k][o]);
                            else acc[o][k] = Elem16<E>::mfma16(fo[o], fi[ks & 1][k], acc[o][k]);
                        }
                        if (ks + 1 < kSteps) {
                            // behind the last instruction that uses fo[o]: its successor; behind the first
                            // instructions of the first NI outer rounds: the inner set of the next step
                            if (k == NI - 1) {
                                if (!kOuterX || x_block_used(o)) fo[o] = __builtin_bit_cast(vec8, load16(st + (base_o ^ ((ks + 1) << kStepShift)) + o * MI * kRowBytes));
                            } else if (k == 0 && o < NI) {
                                if (kOuterX || x_block_used(o)) fi[(ks + 1) & 1][o] = __builtin_bit_cast(vec8, load16(st + (base_i ^ ((ks + 1) << kStepShift)) + o * MI * kRowBytes));
                            }
                        }
                    }
                    if constexpr (COUNT > 0) {
                        if (j >= J0 && (j - J0) % kEvery == 0 && (j - J0) / kEvery < COUNT) issue_one(t, l.sa, l.sb, l.k0, FIRST + (j - J0) / kEvery);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            using Q0 = std::integral_constant<int, 0>; using Q1 = std::integral_constant<int, 1>;
            using Q2 = std::integral_constant<int, 2>; using Q3 = std::integral_constant<int, 3>;
            using NoSync = std::integral_constant<int, -1>;
            static_assert(MI == 16 || TN + TM <= kPerQuarter, "the first quarter of a K step has a matrix instruction for every fragment read");
            if constexpr (kEarlyRelease) {
                // The barrier that frees the stage sits kReleaseAt matrix instructions into the second K step, and
                // all loads of the slice after the next go out behind it, half in each quarter.
                constexpr int L = LA + LB;
                constexpr int AT = kReleaseAt;
                constexpr int M2 = L / 2;
                static_assert(M2 <= kPerQuarter - AT && L - M2 <= kPerQuarter);
                using None = std::integral_constant<int, 0>;
                asm volatile("s_barrier" ::: "memory");   // every wavefront has left the previous tile's epilogue, staged where slice 1 goes
                if (t.k_tiles > 1) issue_range<0, L>(t, smem, 1);
                auto slice = [&](uint32_t kt, auto next_tag, auto next2_tag) {
                    constexpr bool NEXT = decltype(next_tag)::value, NEXT2 = decltype(next2_tag)::value;
                    // this wavefront's loads of slice kt are complete once only those of slice kt+1 are outstanding
                    if constexpr (NEXT) wait_vmcnt<L>();
                    else wait_vmcnt<0>();
                    asm volatile("s_barrier" ::: "memory");   // every wavefront's share of slice kt is in LDS
                    if (kt == 0) after_first_barrier();
                    const char* st = smem + stage_of(t, kt) * kStage;
                    read_fragments(st, 0);
                    quarter(st, Q0{}, SliceLoads{}, None{}, None{}, NoSync{});
                    quarter(st, Q1{}, SliceLoads{}, None{}, None{}, NoSync{});
                    const SliceLoads l2 = NEXT2 ? loads_of(kt + 2) : SliceLoads{};
                    quarter(st, Q2{}, l2, None{}, std::integral_constant<int, NEXT2 ? M2 : 0>{}, std::integral_constant<int, NEXT2 ? AT : -1>{});
                    quarter(st, Q3{}, l2, std::integral_constant<int, M2>{}, std::integral_constant<int, NEXT2 ? L - M2 : 0>{}, NoSync{});
                };
                const uint32_t ahead = t.k_tiles >= 2 ? t.k_tiles - 2 : 0u;   // slices that request slice kt+2
                for (uint32_t kt = 0; kt < ahead; ++kt) slice(kt, std::true_type{}, std::true_type{});
                if (t.k_tiles >= 2) slice(t.k_tiles - 2, std::true_type{}, std::false_type{});
                slice(t.k_tiles - 1, std::false_type{}, std::false_type{});
            } else if constexpr (AHEAD2) {
                static_assert(LA + LB <= kPerQuarter, "the loads of a slice fit behind the matrix instructions of one quarter");
                constexpr int N0 = spread_count(0), N1 = spread_count(1), N2 = spread_count(2), N3 = spread_count(3);
                // Slice 0 was requested by begin(). Every wavefront has left the previous tile's epilogue,
                // which staged its output in the stage slice 1 goes to: its first loads go out here, the
                // others behind the first quarters of slice 0.
                asm volatile("s_barrier" ::: "memory");
                if (t.k_tiles > 1) issue_range<0, N0>(t, smem, 1);
                // One slice: `next_tag` - slice kt+1 exists (its loads N0 .. are issued behind quarters 0 to 2),
                // `next2_tag` - slice kt+2 exists (its first N0 loads go behind the last quarter, into the
                // stage of slice kt, once every wavefront has read its last fragments of it).
                auto slice = [&](uint32_t kt, auto next_tag, auto next2_tag) {
                    constexpr bool NEXT = decltype(next_tag)::value, NEXT2 = decltype(next2_tag)::value;
                    // this wavefront's loads of slice kt are complete once only the first N0 of slice kt+1
                    // are outstanding (the stores of the previous tile's epilogue are older than both)
                    if constexpr (NEXT) wait_vmcnt<N0>();
                    else wait_vmcnt<0>();
                    asm volatile("s_barrier" ::: "memory");   // every wavefront's share of slice kt is in LDS
                    if (kt == 0) after_first_barrier();
                    const char* st = smem + stage_of(t, kt) * kStage;
                    read_fragments(st, 0);
                    const SliceLoads l1 = NEXT ? loads_of(kt + 1) : SliceLoads{};
                    quarter(st, Q0{}, l1, std::integral_constant<int, N0>{}, std::integral_constant<int, NEXT ? N1 : 0>{}, NoSync{});
                    quarter(st, Q1{}, l1, std::integral_constant<int, N0 + N1>{}, std::integral_constant<int, NEXT ? N2 : 0>{}, NoSync{});
                    if constexpr (kEarlyFirst) {
                        const SliceLoads l2 = NEXT2 ? loads_of(kt + 2) : SliceLoads{};
                        quarter(st, Q2{}, l2, std::integral_constant<int, 0>{}, std::integral_constant<int, NEXT2 ? N0 : 0>{},
                                std::integral_constant<int, NEXT2 ? kReleaseAt : -1>{});
                        quarter(st, Q3{}, l2, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, NoSync{});
                        return;
                    }
                    quarter(st, Q2{}, l1, std::integral_constant<int, N0 + N1 + N2>{}, std::integral_constant<int, NEXT ? N3 : 0>{}, NoSync{});
                    if constexpr (NEXT2) {
                        // this wavefront's last reads of the stage have returned; once that holds for every
                        // wavefront the stage takes slice kt+2
                        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
                        asm volatile("s_barrier" ::: "memory");
                    }
                    const SliceLoads l2 = NEXT2 ? loads_of(kt + 2) : SliceLoads{};
                    quarter(st, Q3{}, l2, std::integral_constant<int, 0>{}, std::integral_constant<int, NEXT2 ? N0 : 0>{}, NoSync{});
                };
                const uint32_t ahead = t.k_tiles >= 2 ? t.k_tiles - 2 : 0u;   // slices that request slice kt+2
                for (uint32_t kt = 0; kt < ahead; ++kt) slice(kt, std::true_type{}, std::true_type{});
                if (t.k_tiles >= 2) slice(t.k_tiles - 2, std::true_type{}, std::false_type{});
                slice(t.k_tiles - 1, std::false_type{}, std::false_type{});
            } else {
                static_assert(LA + LB <= kQuarters * kPerQuarter, "the loads of a slice fit behind the matrix instructions of a slice");
                auto top = [&](uint32_t kt) {
                    // This wavefront's loads of slice kt are complete once only those of the later slices
                    // already issued (STAGES-2 of them, fewer at the end of the tile) are outstanding.
                    const uint32_t later = t.k_tiles - 1 - kt;
                    if (STAGES >= 4 && later >= 2) wait_vmcnt<(STAGES >= 4 ? 2 : 0) * kLoadsPerSlice>();
                    else if (STAGES >= 3 && later >= 1) wait_vmcnt<kLoadsPerSlice>();
                    else wait_vmcnt<0>();
                    // every wavefront's share of slice kt is in LDS, and everyone has finished with the stage
                    // the next loads overwrite (slice kt-1, or the previous tile's epilogue staging)
                    asm volatile("s_barrier" ::: "memory");
                    if (kt == 0) after_first_barrier();
                };
                // Quarter q carries the loads q * kPerQuarter ... of the slice STAGES-1 ahead, one behind each
                // matrix instruction, until they run out (sharing them out evenly over the four K steps,
                // which three stages would allow, changes nothing where it was measured: 2.93 against
                // 2.92 ms per forward at the 256-expert top-8 shape, which is bound by HBM)
                auto ksteps = [&](const char* st, const SliceLoads& l, auto loads_tag) {
                    static_for<kQuarters>([&](auto q_tag) {
                        constexpr int q = decltype(q_tag)::value;
                        constexpr int left = LA + LB - q * kPerQuarter;
                        constexpr int count = !decltype(loads_tag)::value || left <= 0 ? 0 : (left < kPerQuarter ? left : kPerQuarter);
                        quarter(st, q_tag, l, std::integral_constant<int, q * kPerQuarter>{}, std::integral_constant<int, count>{}, NoSync{});
                    });
                };
                const uint32_t ahead = t.k_tiles >= uint32_t(STAGES - 1) ? t.k_tiles - (STAGES - 1) : 0u;   // slices that request a later one
                for (uint32_t kt = 0; kt < ahead; ++kt) {
                    top(kt);
                    const char* st = smem + stage_of(t, kt) * kStage;
                    read_fragments(st, 0);
                    ksteps(st, loads_of(kt + STAGES - 1), std::true_type{});
                }
                for (uint32_t kt = ahead; kt < t.k_tiles; ++kt) {
                    top(kt);
                    const char* st = smem + stage_of(t, kt) * kStage;
                    read_fragments(st, 0);
                    ksteps(st, SliceLoads{}, std::false_type{});
                }
            }
        };   // body
        if constexpr (kBlockSkip) {
            // (the same in all lanes of a wavefront; every version goes through the same barriers)
            const int rows_here = int(t.m_valid) - __builtin_amdgcn_readfirstlane(wave) / WAVES_N * WM;
            const int used = rows_here >= WM ? TM : (rows_here <= MI ? 1 : (rows_here + MI - 1) / MI);
            static_assert(TM == 4);
            switch (used) {
                case 1: body(std::integral_constant<int, 1>{}); break;
                case 2: body(std::integral_constant<int, 2>{}); break;
                case 3: body(std::integral_constant<int, 3>{}); break;
                default: body(std::integral_constant<int, 4>{}); break;
            }
        } else {
            body(std::integral_constant<int, TM>{});
        }
    }

    // Whether none of the rows of the wavefronts in row wm of the wavefront grid exist in this tile
    // (the same for all lanes of a wavefront), for the configurations that treat such wavefronts
    // apart: the one with the loads two slices ahead, which runs where experts hold few rows and
    // the loads bound the tile (64-expert shape with skewed routing: 301 against 304 us per forward);
    // where the matrix work bounds it the extra branch costs more than the few such tiles bring
    // (8-expert shape with hidden size 4096: 3.57 against 3.53 ms).
    static __device__ __forceinline__ bool rows_absent(const Tile& t, int wm) {
        if constexpr (AHEAD2) return uint32_t(wm * WM) >= t.m_valid;
        else return false;
    }

    // The stage the tile's last K slice was read from (free once every wavefront has left mainloop()).
    static __device__ __forceinline__ int last_stage(const Tile& t) { return (t.stage0 + t.k_tiles - 1) % STAGES; }
    // The stage the next tile's first slice must go to.
    static __device__ __forceinline__ int next_stage0(const Tile& t) { return (t.stage0 + t.k_tiles) % STAGES; }

    // Epilogue that keeps the fp32 sums as they are (no bias, no activation, no rounding): the
    // tile goes to out[m * ldo + n] as floats, for a caller that sums several K ranges of one product.
    // Every wavefront must have left mainloop(). Each wavefront transposes its 32 x 32 blocks through
    // 4 KB of its own in the stage of the last slice (rows of 128 bytes, chunk c of row r at position
    // c ^ ((r >> 1) & 7)) and stores whole 128-byte lines.
    static __device__ __forceinline__ void finish_partial(const Tile& t, Acc& acc, char* smem, float* out, uint32_t ldo) {
        static_assert(MI == 32, "written for the accumulator layout of the 32 x 32 tiles");
        const uint32_t tid = local_tid();
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int wm = wave / WAVES_N, wn = wave % WAVES_N;
        const int fr_row = lane & 31, fr_half = lane >> 5;
        char* stg = smem + last_stage(t) * kStage + wave * (kPanelRows * 128);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 v{acc[ni][mi][4 * q], acc[ni][mi][4 * q + 1], acc[ni][mi][4 * q + 2], acc[ni][mi][4 * q + 3]};
                    *reinterpret_cast<f32x4*>(stg + fr_row * 128 + (((2 * q + fr_half) ^ ((fr_row >> 1) & 7)) << 4)) = v;
                }
#pragma unroll
                for (int it = 0; it < kPanelRows * 8 / kWave; ++it) {
                    const int id = it * kWave + lane;
                    const int r = id >> 3, c = id & 7;
                    const u32x4 v = load16(stg + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
                    const uint32_t m = wm * WM + mi * 32 + r, n = wn * WN + ni * 32 + c * 4;
                    // the sums are read by other workgroups after a grid-wide barrier
                    if (m < t.m_valid && n < t.n_valid) store16_through(out + size_t(m) * ldo + n, v);
                }
            }
    }

    // Epilogue. Every wavefront must have left mainloop().
    static __device__ __forceinline__ void finish(const Tile& t, Acc& acc, char* smem) {
        if (rows_absent(t, __builtin_amdgcn_readfirstlane(int(local_tid() >> 6)) / WAVES_N)) return;   // nothing of this wavefront's is stored
        const TileOut out{t.c_base, t.ldc, t.m_valid, t.n_valid, t.act};
        epilogue16<E, WM, WN, WAVES_N, STREAM_OUT>(out, acc, smem + last_stage(t) * kStage, smem + kBiasOffset + t.bias_slot * kBiasBytes);
    }
};

// ------------------------------------------------------------------------------------------------
// fp32, matrix cores. 64 x 64 tile, 256 threads = 2 x 2 wavefronts of 32 x 32, K in slices of 16
// through LDS (k-major, rows padded to 68 words: the transposing writes and the operand reads both
// spread over the banks), one 32x32x2 fp32 matrix instruction per two values of K: the weight rows
// are its row operand and the activation rows its column operand, as in the 16-bit tiles, so a
// lane owns 4 consecutive output columns of one output row. K is summed in ascending order, two
// values per instruction - the same order in every launch mode. Serves the fp32 configuration,
// whose sizes are small.
// ------------------------------------------------------------------------------------------------
constexpr int kF32Tile = 64, kF32BK = 16, kF32Pad = 68;
constexpr int gemm_f32_smem_bytes() { return 2 * kF32BK * kF32Pad * 4; }

// T: float, or tf32_t - then the operands lose their lower 13 mantissa bits on the way into LDS
// and the results are rounded to tf32 Elements.
template <int ACT, typename T>
__device__ __forceinline__ void gemm_tile_f32(
    const T* __restrict__ a_elems, const int32_t* __restrict__ a_row_index, uint32_t a_rows, uint32_t lda,
    uint32_t m_valid,
    const T* __restrict__ b_elems, uint32_t ldb, uint32_t n_valid,
    const T* __restrict__ bias_elems, T* __restrict__ c_elems, uint32_t ldc, uint32_t K,
    char* smem) {
    static_assert(sizeof(T) == 4);
    constexpr bool kTf32 = std::is_same<T, tf32_t>::value;
    const float* a_base = reinterpret_cast<const float*>(a_elems);
    const float* b_base = reinterpret_cast<const float*>(b_elems);
    const float* bias = reinterpret_cast<const float*>(bias_elems);
    float* c_base = reinterpret_cast<float*>(c_elems);
    auto operand = [](float v) { return kTf32 ? tf32_operand(v) : v; };
    auto result = [](float v) { return kTf32 ? tf32_round(v) : v; };
    float (*As)[kF32Pad] = reinterpret_cast<float (*)[kF32Pad]>(smem);
    float (*Bs)[kF32Pad] = reinterpret_cast<float (*)[kF32Pad]>(smem + kF32BK * kF32Pad * 4);
    const int tid = threadIdx.x;
    const int ld_row = tid >> 2, ld_kq = tid & 3;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int fr_row = lane & 31, fr_half = lane >> 5;

    const float* pa = nullptr;
    const float* pb = nullptr;
    if (uint32_t(ld_row) < m_valid) {
        // written earlier in the same launch, possibly on another XCD
        uint32_t src = ld_row;
        if (a_row_index) {
            src = uint32_t(load_coherent(a_row_index + ld_row));
            src = src < a_rows ? src : a_rows - 1;
        }
        pa = a_base + size_t(src) * lda + ld_kq * 4;
    }
    if (uint32_t(ld_row) < n_valid) pb = b_base + size_t(ld_row) * ldb + ld_kq * 4;

    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
    for (uint32_t k0 = 0; k0 < K; k0 += kF32BK) {
        const f32x4 va = pa ? *reinterpret_cast<const f32x4*>(pa + k0) : f32x4{0.f, 0.f, 0.f, 0.f};
        const f32x4 vb = pb ? *reinterpret_cast<const f32x4*>(pb + k0) : f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            As[ld_kq * 4 + j][ld_row] = operand(va[j]);
            Bs[ld_kq * 4 + j][ld_row] = operand(vb[j]);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kF32BK; kk += 2) {
            // lanes 0-31 bring K value kk, lanes 32-63 K value kk + 1
            const float w = Bs[kk + fr_half][wn * 32 + fr_row];
            const float x = As[kk + fr_half][wm * 32 + fr_row];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w, x, acc, 0, 0, 0);
        }
    }
    // acc[v]: output row m = wm * 32 + lane % 32, column n = wn * 32 + 8 (v / 4) + 4 (lane / 32) + v % 4
    const uint32_t m = wm * 32 + fr_row;
    if (m < m_valid) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t n0 = wn * 32 + 8 * q + 4 * fr_half;
            float* dst = c_base + size_t(m) * ldc + n0;
            // read by other workgroups later in the same launch: written through the L2
            if (n0 + 4 <= n_valid && ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0)) {
                f32x4 o;
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = result(activate<ACT>(acc[4 * q + j] + bias[n0 + j]));
                store16_through(dst, __builtin_bit_cast(u32x4, o));
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (n0 + j < n_valid) store_through(dst + j, result(activate<ACT>(acc[4 * q + j] + bias[n0 + j])));
            }
        }
    }
}

}  // namespace kleos_amd
