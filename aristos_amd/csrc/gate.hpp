// Gate: logits GEMM fused with softmax, top-k and the per-tile expert histogram, then the
// token-order slot assignment with capacity drop.
//
// Replaces gate::FusedGate / gate::forward of the reference (csrc/include/kleos/moe/gate.cuh:
// 474-720, 729-789). Differences that matter:
//   * one wavefront quad of lanes owns a token, so softmax and top-k are register + cross-lane
//     shuffle work; the reference bounces the accumulator through shared memory to get one
//     thread per token (gate.cuh:560-572);
//   * every expert count is handled inside one workgroup: up to 256 experts with the logits in
//     registers, more in passes of 256 with the logits read back from memory (the reference chains
//     64-expert blocks through global-memory mailboxes, gate.cuh:93-468);
//   * slots are assigned in token order from per-tile histograms and their prefix sums, which
//     makes dropping deterministic; the reference takes a tile's base slot from atomicAdd arrival
//     order (gate.cuh:699).
#pragma once
#include <type_traits>

#include "device_common.hpp"

namespace kleos_amd {

template <typename T>
struct GateK {
    static constexpr int kElemsPer16B = 16 / sizeof(T);
    // K consumed by one mma16_step: each of the 4 lane groups brings 16 bytes
    static constexpr int kStepK = 4 * kElemsPer16B;
};

// Token blocks (16 tokens each) one gate unit works on together: the fragments of the gate weights
// are loaded once per unit and used by every block, which halves the L2 traffic of the weights.
// With 16 expert groups (E > 128) the accumulators of two blocks no longer fit the register file.
// NG = 0 stands for the wide gate (E > 256), which works in passes of 16 groups.
template <int NG>
constexpr int gate_unit_blocks() { return NG == 0 || NG >= 16 ? 1 : 2; }

__host__ __device__ inline uint32_t gate_group_words(uint32_t E, uint32_t k, bool training);
// Softmax, top-k, outputs and histogram of a 16-token tile by a group of four wavefronts (below).
template <typename T, int NL>
__device__ __forceinline__ void gate_group_finish(const LayerParams& p, uint32_t tile, bool valid, f32x4 (&acc)[NL], uint32_t* gsm, uint32_t gtid);
// Up to 64 experts (four groups) and a multiple of four wavefronts: the epilogue of a block is
// shared out over a group of four wavefronts instead of run by one.
template <int NG>
constexpr bool gate_unit_grouped(int kw) { return NG >= 1 && NG <= 4 && kw % 4 == 0; }
// Row stride of the parked partial sums in the grouped epilogue: one word more than a wavefront
// writes, so that the reads, which walk the rows four at a time, spread over all banks.
constexpr int kGateParkStride = kWave + 1;
// LDS floats needed by gate_unit with KW wavefronts: the partial accumulators (4*NG registers of
// 64 lanes) of the KW shares of the hidden dimension of the block being reduced; in the grouped
// epilogue those of both blocks, in padded rows, and the scratch of the groups.
template <int NG>
constexpr int gate_smem_floats(int kw) {
    if (gate_unit_grouped<NG>(kw)) return 2 * kw * NG * 4 * kGateParkStride + (kw / 4) * int(kGateTileTokens * 64 + 64 + kGateTileTokens * 64);
    return kw * (NG == 0 ? 16 : NG) * 4 * kWave;
}
constexpr uint32_t kWideGateMaxK = 32;   // the wide gate keeps a tile's 16 * k picks in LDS

// Softmax, top-k, outputs and the tile histogram of one 16-token tile, run by one wavefront that
// holds the complete logits of the tile: acc[g][v] of lane l is expert 16 g + 4 (l / 16) + v of
// token l % 16.
template <typename T, int NG>
__device__ __forceinline__ void gate_epilogue(const LayerParams& p, uint32_t tile, f32x4 (&acc)[NG], int lane) {
    const int col = lane & 15, chunk = lane >> 4;
    const uint32_t E = p.E;
    const uint32_t token = tile * kGateTileTokens + col;
    // This lane holds, for its token, experts e = 16 g + 4 chunk + v. The logits stay in the
    // accumulator registers (padded experts set to -inf); probabilities are recomputed where they
    // are needed rather than kept, and the selection rounds are packed two to a register: with 16
    // expert groups there is no room for three more arrays of the accumulator's size.
    const float kNegInf = -__builtin_inff();
    float m = kNegInf;
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t e = 16 * g + 4 * chunk + v;
            if (e < E) p.logits[size_t(token) * E + e] = acc[g][v];
            // softmax domain = the E real experts only (gate.cuh:550)
            else acc[g][v] = kNegInf;
            m = fmaxf(m, acc[g][v]);
        }
    m = fmaxf(m, __shfl_xor(m, 16));
    m = fmaxf(m, __shfl_xor(m, 32));
    float d = 0.f;
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) d += __expf(acc[g][v] - m);   // exp(-inf) = 0 for padded experts
    d += __shfl_xor(d, 16);
    d += __shfl_xor(d, 32);
    const float inv_d = 1.0f / d;
    auto prob = [&](float logit) { return __expf(logit - m) * inv_d; };
    T* grow = static_cast<T*>(p.gate_out) + size_t(token) * p.PX;
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t e = 16 * g + 4 * chunk + v;
            // gateOut[t, e] = Element(p) (gate.cuh:590-605); padded columns are zero
            if (e < p.PX) grow[e] = float_to_elem<T>(e < E ? prob(acc[g][v]) : 0.f);
        }
    for (uint32_t e = 16 * NG + 4 * chunk; e < p.PX; e += 16) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
            if (e + v < p.PX) grow[e + v] = float_to_elem<T>(0.f);
    }

    if (p.is_training) {
        // Column sums of the tile's probabilities for the load-balancing loss (gate.cuh:608-635):
        // the 16 tokens of an expert sit in 16 consecutive lanes, summed by a fixed xor tree.
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 16 * g + 4 * chunk + v;
                float col_sum = prob(acc[g][v]);
                col_sum += __shfl_xor(col_sum, 1);
                col_sum += __shfl_xor(col_sum, 2);
                col_sum += __shfl_xor(col_sum, 4);
                col_sum += __shfl_xor(col_sum, 8);
                if (col == 0 && e < E) store_through(p.tile_prob + size_t(tile) * E + e, col_sum);
            }
    }

    // top-k: k rounds of arg-max, equal values go to the lower expert index (gate.cuh:654-670).
    // picked[g][v / 2] holds, in the 16-bit half v % 2, 1 + the round that selected the expert.
    uint32_t picked[NG][2];
#pragma unroll
    for (int g = 0; g < NG; ++g) picked[g][0] = picked[g][1] = 0u;
    auto round_of = [&](int g, int v) { return (picked[g][v >> 1] >> (16 * (v & 1))) & 0xffffu; };
    float den = 0.f;
    constexpr uint32_t kNone = 0x7fffffffu;
    for (uint32_t r = 0; r < p.k; ++r) {
        float best = kNegInf;
        uint32_t bi = kNone;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 16 * g + 4 * chunk + v;
                // padded experts hold -inf and can never beat the initial best
                if (round_of(g, v) == 0 && acc[g][v] > best) {
                    best = acc[g][v];
                    bi = e;
                }
            }
#pragma unroll
        for (int off = 16; off <= 32; off <<= 1) {
            const float ob = __shfl_xor(best, off);
            const uint32_t oi = __shfl_xor(bi, off);
            if (oi != kNone && (bi == kNone || ob > best || (ob == best && oi < bi))) {
                best = ob;
                bi = oi;
            }
        }
        float pv = 0.f;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 16 * g + 4 * chunk + v;
                if (e == bi) {
                    picked[g][v >> 1] |= (r + 1u) << (16 * (v & 1));
                    pv = prob(acc[g][v]);
                }
            }
        // exactly one of the four lanes of this token holds the winner; the others add 0
        pv += __shfl_xor(pv, 16);
        pv += __shfl_xor(pv, 32);
        den += pv;   // mCw, accumulated in selection order (gate.cuh:669)
        if (chunk == 0) {
            store_through(p.topk_expert + size_t(token) * p.k + r, int32_t(bi));
            store_through(p.topk_prob + size_t(token) * p.k + r, pv);
        }
    }
    if (chunk == 0) store_through(p.combine_den + token, den);

    // Histogram of the tile and each token's rank inside it (gate.cuh:678-696).
    uint32_t* super = p.super_count + size_t(p.epoch & 1u) * p.n_super * E +
                      size_t(tile / kSuperTiles) * E;
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t e = 16 * g + 4 * chunk + v;
            const uint32_t rnd = round_of(g, v);
            const bool sel = rnd != 0;
            const unsigned long long mask = __ballot(sel);
            const uint32_t sub = uint32_t(mask >> (16 * chunk)) & 0xffffu;
            if (sel)
                store_through(p.topk_slot + size_t(token) * p.k + (rnd - 1), int32_t(__popc(sub & ((1u << col) - 1u))));
            if (col == 0 && e < E) {
                const uint32_t cnt = __popc(sub);
                store_through(p.tile_count + size_t(tile) * E + e, cnt);
                if (cnt) atomic_add_agent(super + e, cnt);
            }
        }
}

// One gate unit: gate_unit_blocks<NG>() consecutive 16-token tiles, computed by the KW wavefronts of the
// workgroup, which split the hidden dimension. Wavefront b then reduces the partial sums of block
// b in a fixed order and runs its epilogue. Every thread of the workgroup must call the function
// (it contains workgroup barriers); `smem` holds gate_smem_floats<NG>(KW) floats and may be reused
// after the call.
template <typename T, int NG, int KW>
__device__ __forceinline__ void gate_unit(const LayerParams& p, uint32_t unit, float* smem) {
    constexpr int TB = gate_unit_blocks<NG>();
    static_assert(TB <= KW);
    const int wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    const int col = lane & 15;       // token inside a block / expert row inside a group
    const int chunk = lane >> 4;     // which 16-byte K chunk of a step this lane loads
    const uint32_t H = p.H;
    constexpr int kStepK = GateK<T>::kStepK;
    constexpr int kPer = GateK<T>::kElemsPer16B;
    const uint32_t steps = H / kStepK;
    // Wavefront w works on share (w + unit / 8) % KW of the hidden dimension: the units that run on
    // one XCD at the same time (unit numbers 8 apart) then ask its L2 for different lines of the
    // gate weights at any moment instead of all for the same ones.
    const uint32_t part = (uint32_t(wave) + (unit >> 3)) % uint32_t(KW);
    const uint32_t s0 = (steps * part) / KW, s1 = (steps * (part + 1)) / KW;

    const T* xrow[TB];
    bool live[TB];
#pragma unroll
    for (int b = 0; b < TB; ++b) {
        const uint32_t tile = unit * TB + b;
        live[b] = tile < p.n_gate_tiles;
        // a block past the end re-reads the last tile; nothing of it is written
        const uint32_t token = (live[b] ? tile : p.n_gate_tiles - 1) * kGateTileTokens + col;
        xrow[b] = static_cast<const T*>(p.x) + size_t(token) * H + chunk * kPer;
    }
    const T* wrow = static_cast<const T*>(p.wg) + size_t(col) * H + chunk * kPer;

    f32x4 acc[TB][NG];
#pragma unroll
    for (int b = 0; b < TB; ++b)
#pragma unroll
        for (int g = 0; g < NG; ++g) acc[b][g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // logits^T: experts are the matrix-core rows, tokens its columns (gate.cuh:526-534). The loads
    // of U steps are in flight together: the activation rows stream from HBM once and this is what
    // keeps enough of them in flight. They are issued in halves of U / 2 steps, and a half is
    // requested again (for U steps further on) as soon as its matrix instructions have read it, so
    // the memory pipeline never runs empty between one batch and the next (worth 0.5 us of 12.5 per
    // workgroup at the 64-expert shape with a hidden size of 2048: the loop runs at what a CU gets
    // of the memory system while all CUs stream, about 32 GB/s).
    constexpr int U = NG <= 2 ? 8 : (NG <= 4 ? 4 : (NG <= 8 ? 2 : 1));
    constexpr int UH = U >= 2 ? U / 2 : 1;
    uint32_t s = s0;
    if constexpr (U >= 2) {
        u32x4 xb[U][TB], wa[U][NG];
        auto issue = [&](auto first_slot, uint32_t s_first) {
            constexpr int u0 = decltype(first_slot)::value;
#pragma unroll
            for (int u = 0; u < UH; ++u) {
                const uint32_t off = (s_first + u) * kStepK;
#pragma unroll
                for (int b = 0; b < TB; ++b) xb[u0 + u][b] = load16(xrow[b] + off);
#pragma unroll
                for (int g = 0; g < NG; ++g) wa[u0 + u][g] = load16(wrow + size_t(g) * 16 * H + off);
            }
            __builtin_amdgcn_sched_barrier(0);   // the loads stay where they are written
        };
        auto consume = [&](auto first_slot) {
            constexpr int u0 = decltype(first_slot)::value;
#pragma unroll
            for (int u = 0; u < UH; ++u)
#pragma unroll
                for (int g = 0; g < NG; ++g)
#pragma unroll
                    for (int b = 0; b < TB; ++b) acc[b][g] = mma16_step(wa[u0 + u][g], xb[u0 + u][b], acc[b][g], T{});
            __builtin_amdgcn_sched_barrier(0);
        };
        constexpr std::integral_constant<int, 0> lower{};
        constexpr std::integral_constant<int, UH> upper{};
        if (s + U <= s1) {
            issue(lower, s);
            issue(upper, s + UH);
            for (; s + 2 * U <= s1; s += U) {
                consume(lower);
                issue(lower, s + U);
                consume(upper);
                issue(upper, s + U + UH);
            }
            consume(lower);
            consume(upper);
            s += U;
        }
    }
    for (; s < s1; ++s) {
        const uint32_t off = s * kStepK;
        u32x4 xb[TB];
#pragma unroll
        for (int b = 0; b < TB; ++b) xb[b] = load16(xrow[b] + off);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const u32x4 a = load16(wrow + size_t(g) * 16 * H + off);
#pragma unroll
            for (int b = 0; b < TB; ++b) acc[b][g] = mma16_step(a, xb[b], acc[b][g], T{});
        }
    }

    if constexpr (gate_unit_grouped<NG>(KW)) {
        // Every wavefront parks the partial sums of its share of both blocks in LDS; block b then
        // belongs to group b of four wavefronts (one group: block after block), 16 lanes per token
        // and four experts per lane, which add the shares in ascending order (a fixed order: the
        // logits depend neither on timing nor on which wavefront worked on which share).
        static_assert(TB == 2);
        constexpr int kShare = NG * 4 * kGateParkStride;
#pragma unroll
        for (int b = 0; b < TB; ++b) {
            float* dst = smem + (b * KW + part) * kShare;
#pragma unroll
            for (int g = 0; g < NG; ++g)
#pragma unroll
                for (int v = 0; v < 4; ++v) dst[(g * 4 + v) * kGateParkStride + lane] = acc[b][g][v];
        }
        __syncthreads();
        constexpr int kGroups = KW / 4;
        const uint32_t group = uint32_t(wave) >> 2, gtid = threadIdx.x & 255u;
        uint32_t* gsm = reinterpret_cast<uint32_t*>(smem + TB * KW * kShare) + group * gate_group_words(p.E, p.k, p.is_training != 0);
        const int sub = lane & 15;                              // experts 4 sub .. 4 sub + 3
        const int tl = 4 * (wave & 3) + (lane >> 4);            // token inside the block
#pragma unroll
        for (int b0 = 0; b0 < TB; b0 += kGroups) {
            const uint32_t b = b0 + group;
            const uint32_t tile = unit * TB + b;
            const bool valid = b < uint32_t(TB) && tile < p.n_gate_tiles;
            f32x4 sum[1] = {f32x4{0.f, 0.f, 0.f, 0.f}};
            if (valid && sub < 4 * NG) {
                // expert 4 sub + v sits in row 4 (sub / 4) + v of a share, at lane 16 (sub % 4) + token
                const float* src = smem + (b * KW) * kShare + ((sub >> 2) * 4) * kGateParkStride + 16 * (sub & 3) + tl;
#pragma unroll
                for (int v = 0; v < 4; ++v) sum[0][v] = src[v * kGateParkStride];
#pragma unroll
                for (int w = 1; w < KW; ++w)
#pragma unroll
                    for (int v = 0; v < 4; ++v) sum[0][v] += src[w * kShare + v * kGateParkStride];
            }
            gate_group_finish<T, 1>(p, tile, valid, sum, gsm, gtid);
        }
        return;
    }
    // Block b: every wavefront parks the partial sums of its share in LDS, wavefront b adds them
    // in ascending order of the shares (a fixed order: the logits depend neither on timing nor on
    // which wavefront worked on which share).
#pragma unroll
    for (int b = 0; b < TB; ++b) {
        float* dst = smem + part * (NG * 4 * kWave);
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) dst[(g * 4 + v) * kWave + lane] = acc[b][g][v];
        __syncthreads();
        if (wave == b) {
#pragma unroll
            for (int g = 0; g < NG; ++g)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[b][g][v] = smem[(g * 4 + v) * kWave + lane];
#pragma unroll
            for (int w = 1; w < KW; ++w) {
                const float* src = smem + w * (NG * 4 * kWave);
#pragma unroll
                for (int g = 0; g < NG; ++g)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[b][g][v] += src[(g * 4 + v) * kWave + lane];
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int b = 0; b < TB; ++b)
        if (wave == b && live[b]) gate_epilogue<T, NG>(p, unit * TB + b, acc[b], lane);
    __syncthreads();
}

template <typename T>
__device__ __forceinline__ void gate_wide_epilogue(const LayerParams& p, uint32_t tile, float* smem, int lane);

// The gate for more than 256 experts: one 16-token block per unit, the experts in passes of 256.
// Every pass is the K loop and the reduction of gate_unit with 16 groups; wavefront 0 stores the
// pass's logits, and when all passes are done it reads them back for softmax and top-k (each lane
// reads exactly the words it stored). Selection needs no record of what was picked: round r takes
// the largest logit that comes after the previous pick in the order (logit descending, expert
// ascending), which is the same k rounds of arg-max with ties to the lower index
// (gate.cuh:654-670). The tile's picks go through LDS for the in-tile ranks and the histogram.
// Every thread of the workgroup must call the function; `smem` holds gate_smem_floats<0>(KW) floats.
template <typename T, int KW>
__device__ __forceinline__ void gate_unit_wide(const LayerParams& p, uint32_t unit, float* smem) {
    constexpr int NG = 16;
    const int wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    const int col = lane & 15, chunk = lane >> 4;
    const uint32_t H = p.H, E = p.E;
    constexpr int kStepK = GateK<T>::kStepK;
    constexpr int kPer = GateK<T>::kElemsPer16B;
    const uint32_t steps = H / kStepK;
    const uint32_t part = (uint32_t(wave) + (unit >> 3)) % uint32_t(KW);
    const uint32_t s0 = (steps * part) / KW, s1 = (steps * (part + 1)) / KW;
    const uint32_t tile = unit;
    const bool live = tile < p.n_gate_tiles;
    const uint32_t token = (live ? tile : p.n_gate_tiles - 1) * kGateTileTokens + col;
    const T* xrow = static_cast<const T*>(p.x) + size_t(token) * H + chunk * kPer;
    float* my_logits = p.logits + size_t(token) * E;

    for (uint32_t e0 = 0; e0 < E; e0 += 16 * NG) {
        f32x4 acc[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
        // weight rows past the padded expert count re-read its last row; their logits are never stored
        auto wrow = [&](int g) {
            const uint32_t r = e0 + 16 * g + col;
            return static_cast<const T*>(p.wg) + size_t(r < p.PX ? r : p.PX - 1) * H + chunk * kPer;
        };
        // the loads of U steps are issued together before their matrix instructions
        constexpr int U = 2;
        uint32_t s = s0;
        for (; s + U <= s1; s += U) {
            u32x4 xb[U], wa[U][NG];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t off = (s + u) * kStepK;
                xb[u] = load16(xrow + off);
#pragma unroll
                for (int g = 0; g < NG; ++g) wa[u][g] = load16(wrow(g) + off);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int g = 0; g < NG; ++g) acc[g] = mma16_step(wa[u][g], xb[u], acc[g], T{});
        }
        for (; s < s1; ++s) {
            const uint32_t off = s * kStepK;
            const u32x4 xb = load16(xrow + off);
#pragma unroll
            for (int g = 0; g < NG; ++g) acc[g] = mma16_step(load16(wrow(g) + off), xb, acc[g], T{});
        }
        float* dst = smem + part * (NG * 4 * kWave);
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) dst[(g * 4 + v) * kWave + lane] = acc[g][v];
        __syncthreads();
        if (wave == 0 && live) {
#pragma unroll
            for (int g = 0; g < NG; ++g)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float sum = smem[(g * 4 + v) * kWave + lane];
#pragma unroll
                    for (int w = 1; w < KW; ++w) sum += smem[w * (NG * 4 * kWave) + (g * 4 + v) * kWave + lane];
                    const uint32_t e = e0 + 16 * g + 4 * chunk + v;
                    if (e < E) my_logits[e] = sum;
                }
        }
        __syncthreads();
    }

    if (wave == 0 && live) gate_wide_epilogue<T>(p, tile, smem, lane);
    __syncthreads();
}

// Softmax, top-k, outputs and the tile histogram of one 16-token tile whose logits are in memory
// (p.logits), run by one wavefront; `smem` holds E + 16 k words private to it. A lane reads the
// logits it (or the wavefront that runs this) stored itself, or ones stored before a grid-wide
// barrier: device-coherent loads either way.
template <typename T>
__device__ __forceinline__ void gate_wide_epilogue(const LayerParams& p, uint32_t tile, float* smem, int lane) {
    const int col = lane & 15, chunk = lane >> 4;
    const uint32_t E = p.E, k = p.k;
    const uint32_t token = tile * kGateTileTokens + col;
    float* my_logits = p.logits + size_t(token) * E;
    {
        // lane (col, chunk) owns experts 16 j + 4 chunk + v of token col, as in the register gate
        const float kNegInf = -__builtin_inff();
        const uint32_t groups = (E + 15) / 16;
        auto logit = [&](uint32_t e) { return load_coherent(my_logits + e); };
        float m = kNegInf;
        for (uint32_t j = 0; j < groups; ++j)
#pragma unroll
            for (uint32_t v = 0; v < 4; ++v) {
                const uint32_t e = 16 * j + 4 * chunk + v;
                if (e < E) m = fmaxf(m, logit(e));
            }
        m = fmaxf(m, __shfl_xor(m, 16));
        m = fmaxf(m, __shfl_xor(m, 32));
        float d = 0.f;
        for (uint32_t j = 0; j < groups; ++j)
#pragma unroll
            for (uint32_t v = 0; v < 4; ++v) {
                const uint32_t e = 16 * j + 4 * chunk + v;
                if (e < E) d += __expf(logit(e) - m);
            }
        d += __shfl_xor(d, 16);
        d += __shfl_xor(d, 32);
        const float inv_d = 1.0f / d;
        auto prob = [&](float l) { return __expf(l - m) * inv_d; };
        T* grow = static_cast<T*>(p.gate_out) + size_t(token) * p.PX;
        for (uint32_t j = 0; 16 * j < p.PX; ++j)
#pragma unroll
            for (uint32_t v = 0; v < 4; ++v) {
                const uint32_t e = 16 * j + 4 * chunk + v;
                const float pe = e < E ? prob(logit(e)) : 0.f;
                if (e < p.PX) grow[e] = float_to_elem<T>(pe);   // padded columns are zero (gate.cuh:590-605)
                if (p.is_training) {
                    // column sum over the tile's 16 tokens, a fixed xor tree (gate.cuh:608-635)
                    float col_sum = pe;
                    col_sum += __shfl_xor(col_sum, 1);
                    col_sum += __shfl_xor(col_sum, 2);
                    col_sum += __shfl_xor(col_sum, 4);
                    col_sum += __shfl_xor(col_sum, 8);
                    if (col == 0 && e < E) store_through(p.tile_prob + size_t(tile) * E + e, col_sum);
                }
            }

        uint32_t* s_hist = reinterpret_cast<uint32_t*>(smem);   // [E] tokens of the tile routed to e
        uint32_t* s_sel = s_hist + E;                           // [16][k] the tile's picks
        for (uint32_t e = lane; e < E; e += kWave) s_hist[e] = 0u;
        constexpr uint32_t kNone = 0x7fffffffu;
        float den = 0.f, prev_l = 0.f;
        uint32_t prev_e = 0;
        for (uint32_t r = 0; r < k; ++r) {
            float best = kNegInf;
            uint32_t bi = kNone;
            for (uint32_t j = 0; j < groups; ++j)
#pragma unroll
                for (uint32_t v = 0; v < 4; ++v) {
                    const uint32_t e = 16 * j + 4 * chunk + v;
                    if (e >= E) continue;
                    const float l = logit(e);
                    const bool open = r == 0 || l < prev_l || (l == prev_l && e > prev_e);
                    if (open && (bi == kNone || l > best)) {
                        best = l;
                        bi = e;
                    }
                }
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const float ob = __shfl_xor(best, off);
                const uint32_t oi = __shfl_xor(bi, off);
                if (oi != kNone && (bi == kNone || ob > best || (ob == best && oi < bi))) {
                    best = ob;
                    bi = oi;
                }
            }
            // all four lanes of the token hold the pick now
            const float pv = bi != kNone ? prob(best) : 0.f;
            den += pv;   // mCw, accumulated in selection order (gate.cuh:669)
            prev_l = best;
            prev_e = bi;
            if (chunk == 0) {
                store_through(p.topk_expert + size_t(token) * k + r, int32_t(bi));
                store_through(p.topk_prob + size_t(token) * k + r, pv);
                s_sel[uint32_t(col) * k + r] = bi;
            }
        }
        if (chunk == 0) store_through(p.combine_den + token, den);
        // in-tile rank of every pick and the tile histogram (gate.cuh:678-696); the LDS operations of
        // one wavefront complete in order, so the picks written above are visible here
        uint32_t* super = p.super_count + size_t(p.epoch & 1u) * p.n_super * E + size_t(tile / kSuperTiles) * E;
        const uint32_t pairs = kGateTileTokens * k;
        for (uint32_t i = lane; i < pairs; i += kWave) {
            const uint32_t t = i / k, e = s_sel[i];
            uint32_t before = 0, total = 0;
            for (uint32_t o = 0; o < pairs; ++o) {
                const bool same = s_sel[o] == e;
                total += same;
                before += same && o / k < t;
            }
            store_through(p.topk_slot + ((size_t(tile) * kGateTileTokens + t) * k + (i % k)), int32_t(before));
            if (before == 0 && e < E) s_hist[e] = total;   // one writer: the first token that picked e
        }
        for (uint32_t e = lane; e < E; e += kWave) {
            const uint32_t cnt = s_hist[e];
            store_through(p.tile_count + size_t(tile) * E + e, cnt);
            if (cnt) atomic_add_agent(super + e, cnt);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Gate of the 16-bit Elements with more than 64 experts: the logits come from a tiled product
// (128 tokens x 256 experts per workgroup, the hidden dimension split into p.gate_splits ranges
// whose fp32 sums land in p.gate_partial[split][token][PX]), so the gate weights are read once per
// 128 tokens instead of once per 16 or 32. After a grid-wide barrier the 16-token tiles are
// reduced - by a group of four wavefronts each up to 256 experts, by one wavefront above: the
// ranges are added in ascending order (a fixed order: the logits do not depend on timing or on the
// launch mode), then softmax, top-k and the tile's histogram as in the other gates.
// ------------------------------------------------------------------------------------------------
// The sum over the ranges of the 4 experts e0 .. e0+3 of `token` (e0 a multiple of 4; experts past
// the padded count read as 0).
__device__ __forceinline__ f32x4 gate_partial_sum(const LayerParams& p, coherent_rows_t partial, uint32_t token, uint32_t e0) {
    f32x4 sum{0.f, 0.f, 0.f, 0.f};
    if (e0 < p.PX) {
        for (uint32_t s = 0; s < p.gate_splits; ++s) {
            const uint32_t offset = ((s * p.S + token) * p.PX + e0) * 4u;
            sum += __builtin_bit_cast(f32x4, load16_coherent(partial, offset));
        }
    }
    return sum;
}

// Up to 256 experts, a tile worked on by a group of four wavefronts (256 threads): wavefront w of
// the group takes tokens 4 w .. 4 w + 3 of the tile, 16 lanes per token, each lane the experts
// 64 j + 4 (lane % 16) + v (j < NL, NL * 64 >= PX, v < 4). Against one wavefront per tile every per-lane
// loop over the experts is four times shorter, and the partial sums, logits and gate outputs move
// in runs of 256 and 128 bytes per token. The tile's picks meet in LDS: every pick counts the picks
// of its expert by earlier tokens for its in-tile rank and adds itself to the tile's histogram,
// which the group then writes out. Same sums over the
// ranges, same selection rule and same order of the denominator as gate_epilogue; the softmax
// denominator is summed in a different (fixed) order.
// `gsm`: gate_group_words(p) words of LDS private to the group. Every thread of the workgroup must
// call the function the same number of times (it contains workgroup barriers); a group without a
// tile passes valid = false.
__host__ __device__ inline uint32_t gate_group_words(uint32_t E, uint32_t k, bool training) {
    return kGateTileTokens * k + E + (training ? kGateTileTokens * E : 0u);
}
template <typename T, int NL>
__device__ __forceinline__ void gate_reduce_group(const LayerParams& p, uint32_t tile, bool valid, uint32_t* gsm, uint32_t gtid) {
    const int lane = gtid & 63, sub = lane & 15;
    const uint32_t tl = 4 * (gtid >> 6) + (lane >> 4);
    f32x4 acc[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (valid) {
        const uint32_t token = tile * kGateTileTokens + tl;
        const coherent_rows_t partial = coherent_rows(p.gate_partial);
        // range by range, in ascending order; the loads of two ranges in flight together
        for (uint32_t s0 = 0; s0 < p.gate_splits; s0 += 2) {
            u32x4 v[2][NL];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const uint32_t s = s0 + u < p.gate_splits ? s0 + u : s0;
                const uint32_t row = ((s * p.S + token) * p.PX + 4 * sub) * 4u;
#pragma unroll
                for (int j = 0; j < NL; ++j) v[u][j] = uint32_t(64 * j) < p.PX ? load16_coherent(partial, row + 256u * j) : u32x4{0, 0, 0, 0};
            }
#pragma unroll
            for (int j = 0; j < NL; ++j) acc[j] += __builtin_bit_cast(f32x4, v[0][j]);
            if (s0 + 1 < p.gate_splits) {
#pragma unroll
                for (int j = 0; j < NL; ++j) acc[j] += __builtin_bit_cast(f32x4, v[1][j]);
            }
        }
    }
    gate_group_finish<T, NL>(p, tile, valid, acc, gsm, gtid);
}

// The part of the group's work that follows the logits: `acc[j][v]` of a lane is the logit of expert
// 64 j + 4 (lane % 16) + v of its token (anything for experts past the padded count).
template <typename T, int NL>
__device__ __forceinline__ void gate_group_finish(const LayerParams& p, uint32_t tile, bool valid, f32x4 (&acc)[NL], uint32_t* gsm, uint32_t gtid) {
    constexpr uint32_t kGroupThreads = 4 * kWave;
    const int lane = gtid & 63, sub = lane & 15;
    const uint32_t gw = gtid >> 6, tl = 4 * gw + (lane >> 4);
    const uint32_t E = p.E, k = p.k;
    uint32_t* s_sel = gsm;                                   // [16][k] expert picked by token t in round r
    uint32_t* s_hist = gsm + kGateTileTokens * k;            // [E]
    float* s_prob = reinterpret_cast<float*>(s_hist + E);    // [16][E], training only
    for (uint32_t e = gtid; e < E; e += kGroupThreads) s_hist[e] = 0u;
    if (valid) {
        const uint32_t token = tile * kGateTileTokens + tl;
        const float kNegInf = -__builtin_inff();
        float m = kNegInf;
        const bool whole_quads = (E & 3u) == 0u;   // a lane's four experts are all real or all padding
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const uint32_t e0 = 64 * j + 4 * sub;
            if (whole_quads && e0 < E) *reinterpret_cast<f32x4*>(p.logits + size_t(token) * E + e0) = acc[j];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = e0 + v;
                if (e >= E) acc[j][v] = kNegInf;   // softmax domain = the E real experts only (gate.cuh:550)
                else if (!whole_quads) p.logits[size_t(token) * E + e] = acc[j][v];
                m = fmaxf(m, acc[j][v]);
            }
        }
        m = row16_allreduce(m, [](float a, float b) { return fmaxf(a, b); });
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < NL; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) d += __expf(acc[j][v] - m);
        d = row16_allreduce(d, [](float a, float b) { return a + b; });
        const float inv_d = 1.0f / d;
        auto prob = [&](float logit) { return __expf(logit - m) * inv_d; };
        // gateOut[t, e] = Element(p) (gate.cuh:590-605); padded columns are zero
        T* grow = static_cast<T*>(p.gate_out) + size_t(token) * p.PX;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            T o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 64 * j + 4 * sub + v;
                o[v] = float_to_elem<T>(e < E ? prob(acc[j][v]) : 0.f);
                if (p.is_training && e < E) s_prob[tl * E + e] = prob(acc[j][v]);
            }
            // the padded row length is a multiple of 64: the four columns are inside the row together
            using Quad = std::conditional_t<sizeof(T) == 2, uint2, f32x4>;
            static_assert(sizeof(Quad) == 4 * sizeof(T));
            Quad raw;
            __builtin_memcpy(&raw, o, sizeof(Quad));
            if (uint32_t(64 * j) < p.PX) *reinterpret_cast<Quad*>(grow + 64 * j + 4 * sub) = raw;
        }
        // top-k: k rounds of arg-max, equal values go to the lower expert index (gate.cuh:654-670);
        // a picked expert leaves the working copy
        f32x4 w[NL];
#pragma unroll
        for (int j = 0; j < NL; ++j) w[j] = acc[j];
        float den = 0.f;
        constexpr uint32_t kNone = 0x7fffffffu;
        for (uint32_t r = 0; r < k; ++r) {
            float best = kNegInf;
            uint32_t bi = kNone;
#pragma unroll
            for (int j = 0; j < NL; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (w[j][v] > best) {
                        best = w[j][v];
                        bi = 64 * j + 4 * sub + v;
                    }
            // (the rule is symmetric in the two candidates, so the lanes of a pair agree after a step)
            auto better = [&](float ob, uint32_t oi) {
                if (oi != kNone && (bi == kNone || ob > best || (ob == best && oi < bi))) {
                    best = ob;
                    bi = oi;
                }
            };
            { const float ob = row16_peer<0>(best); const uint32_t oi = row16_peer<0>(bi); better(ob, oi); }
            { const float ob = row16_peer<1>(best); const uint32_t oi = row16_peer<1>(bi); better(ob, oi); }
            { const float ob = row16_peer<2>(best); const uint32_t oi = row16_peer<2>(bi); better(ob, oi); }
            { const float ob = row16_peer<3>(best); const uint32_t oi = row16_peer<3>(bi); better(ob, oi); }
            // every lane of the token knows the winner and its logit
            const float pv = bi != kNone ? prob(best) : 0.f;
            den += pv;   // mCw, accumulated in selection order (gate.cuh:669)
#pragma unroll
            for (int j = 0; j < NL; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (uint32_t(64 * j + 4 * sub + v) == bi) w[j][v] = kNegInf;
            if (sub == 0) {
                store_through(p.topk_expert + size_t(token) * k + r, int32_t(bi));
                store_through(p.topk_prob + size_t(token) * k + r, pv);
                s_sel[tl * k + r] = bi;
            }
        }
        if (sub == 0) store_through(p.combine_den + token, den);
    }
    __syncthreads();
    // in-tile ranks (gate.cuh:678-696): pick r of token t ranks behind the picks of the same expert
    // by the tokens before t (a token's own picks are distinct experts). One pick per thread, the
    // earlier picks read four at a time (every lane reads the same words: broadcasts); the reads
    // may run up to three words past the picks of the earlier tokens, which stays inside the
    // group's LDS and is masked out.
    if (valid) {
        for (uint32_t i = gtid; i < kGateTileTokens * k; i += kGroupThreads) {
            const uint32_t e = s_sel[i];
            const uint32_t before = (i / k) * k;
            uint32_t rank = 0;
            if (e < E) {
                for (uint32_t j = 0; j < before; j += 4) {
                    const uint32_t a = s_sel[j], b = s_sel[j + 1], c = s_sel[j + 2], d = s_sel[j + 3];
                    rank += uint32_t(a == e) + uint32_t(b == e && j + 1 < before) + uint32_t(c == e && j + 2 < before) +
                            uint32_t(d == e && j + 3 < before);
                }
                atomicAdd(s_hist + e, 1u);
            }
            store_through(p.topk_slot + size_t(tile) * kGateTileTokens * k + i, int32_t(rank));
        }
    }
    __syncthreads();
    if (valid) {
        uint32_t* super = p.super_count + size_t(p.epoch & 1u) * p.n_super * E + size_t(tile / kSuperTiles) * E;
        for (uint32_t e = gtid; e < E; e += kGroupThreads) {
            const uint32_t cnt = s_hist[e];
            store_through(p.tile_count + size_t(tile) * E + e, cnt);
            if (cnt) atomic_add_agent(super + e, cnt);
            if (p.is_training) {
                // column sums of the tile's probabilities for the load-balancing loss (gate.cuh:608-635)
                float col_sum = 0.f;
                for (uint32_t t = 0; t < kGateTileTokens; ++t) col_sum += s_prob[t * E + e];
                store_through(p.tile_prob + size_t(tile) * E + e, col_sum);
            }
        }
    }
    __syncthreads();   // the next tile clears the histogram
}

// More than 256 experts: the sums go to p.logits, which the epilogue for many experts reads back.
// `smem` holds E + 16 k words private to the calling wavefront.
template <typename T>
__device__ __forceinline__ void gate_reduce_tile_wide(const LayerParams& p, uint32_t tile, float* smem, int lane) {
    const int col = lane & 15, chunk = lane >> 4;
    const uint32_t token = tile * kGateTileTokens + col;
    const coherent_rows_t partial = coherent_rows(p.gate_partial);
    for (uint32_t e0 = 4 * chunk; e0 < p.E; e0 += 16) {
        const f32x4 sum = gate_partial_sum(p, partial, token, e0);
#pragma unroll
        for (uint32_t v = 0; v < 4; ++v)
            if (e0 + v < p.E) p.logits[size_t(token) * p.E + e0 + v] = sum[v];
    }
    gate_wide_epilogue<T>(p, tile, smem, lane);
}

// Slot assignment for one 16-token tile per wavefront. Every thread of the workgroup must call it
// (it contains workgroup barriers); a wave without work passes valid = false. `base` is LDS
// scratch of E uint32 private to the calling wave. Must run after every gate tile has finished
// and released its results; what the gate tiles wrote is read with device-coherent loads.
//   slot = (tokens routed to e in all earlier tiles) + (rank inside this tile); a token keeps its
//   expert iff slot < EC (gate.cuh:710-716).
__device__ __forceinline__ void slot_tile(const LayerParams& p, uint32_t tile, bool valid,
                                          uint32_t* base) {
    const int lane = threadIdx.x & 63;
    const uint32_t E = p.E;
    const uint32_t* super = p.super_count + size_t(p.epoch & 1u) * p.n_super * E;
    // The tile's (token, expert) pairs are requested first: they do not depend on the counts, and
    // every dependent round trip to memory written by other XCDs costs more than a microsecond.
    const uint32_t pairs = kGateTileTokens * p.k;
    constexpr uint32_t kInline = 4;            // pairs per lane kept in registers (k <= 16)
    uint32_t pe[kInline];
    int32_t pr[kInline];
#pragma unroll
    for (uint32_t u = 0; u < kInline; ++u) {
        const uint32_t i = lane + u * kWave;
        pe[u] = 0; pr[u] = 0;
        if (valid && i < pairs) {
            pe[u] = uint32_t(load_coherent(p.topk_expert + size_t(tile) * pairs + i));
            pr[u] = load_coherent(p.topk_slot + size_t(tile) * pairs + i);
        }
    }
    if (valid) {
        const uint32_t sup = tile / kSuperTiles;
        const uint32_t first = sup * kSuperTiles;
        // The coarse rows before this tile's block and the tile rows inside it form one list of
        // n rows, summed per expert in batches of 16 loads that are in flight together (the row
        // index is clamped instead of branching, so the loads of a batch issue back to back).
        const uint32_t n = sup + (tile - first);
        auto row_ptr = [&](uint32_t r) {
            return r < sup ? super + size_t(r) * E : p.tile_count + size_t(first + (r - sup)) * E;
        };
        for (uint32_t e = lane; e < E; e += kWave) {
            uint32_t acc = 0;
            constexpr uint32_t kBatch = 16;
            for (uint32_t r0 = 0; r0 < n; r0 += kBatch) {
                uint32_t v[kBatch];
#pragma unroll
                for (uint32_t u = 0; u < kBatch; ++u) v[u] = load_coherent(row_ptr(r0 + u < n ? r0 + u : n - 1) + e);
#pragma unroll
                for (uint32_t u = 0; u < kBatch; ++u) acc += r0 + u < n ? v[u] : 0u;
            }
            base[e] = acc;
            // training: the wavefront of a block's first tile also sums the block's probability rows
            if (p.is_training && tile == first) {
                const uint32_t rows = p.n_gate_tiles - first < uint32_t(kSuperTiles) ? p.n_gate_tiles - first
                                                                                      : uint32_t(kSuperTiles);
                float total = 0.f;
                for (uint32_t r0 = 0; r0 < rows; r0 += 16) {
                    float v[16];
#pragma unroll
                    for (uint32_t u = 0; u < 16; ++u)
                        v[u] = load_coherent(p.tile_prob + size_t(first + (r0 + u < rows ? r0 + u : rows - 1)) * E + e);
#pragma unroll
                    for (uint32_t u = 0; u < 16; ++u) total += r0 + u < rows ? v[u] : 0.f;
                }
                store_through(p.super_prob + size_t(sup) * E + e, total);
            }
            // total routed per expert, dropped tokens included (the reference's eC, gate.cuh:699)
            if (tile + 1 == p.n_gate_tiles)
                store_through(p.expert_count + e, acc + load_coherent(p.tile_count + size_t(tile) * E + e));
        }
    }
    __syncthreads();
    if (valid) {
        auto assign = [&](uint32_t i, uint32_t e, int32_t rank) {
            const size_t idx = size_t(tile) * pairs + i;
            const uint32_t token = tile * kGateTileTokens + i / p.k;
            if (e >= E) e = E - 1;   // cannot happen; keeps every address below inside its table
            const uint32_t slot = base[e] + uint32_t(rank);
            const bool keep = slot < p.EC && slot < p.cap_rows;
            store_through(p.topk_slot + idx, keep ? int32_t(slot) : -1);
            if (keep) store_through(p.slot_token + size_t(e) * p.cap_rows + slot, int32_t(token));
        };
#pragma unroll
        for (uint32_t u = 0; u < kInline; ++u)
            if (lane + u * kWave < pairs) assign(lane + u * kWave, pe[u], pr[u]);
        for (uint32_t i = lane + kInline * kWave; i < pairs; i += kWave)
            assign(i, uint32_t(load_coherent(p.topk_expert + size_t(tile) * pairs + i)),
                   load_coherent(p.topk_slot + size_t(tile) * pairs + i));
    }
    __syncthreads();
}

// Training mode, one wavefront, after the slot phase has been released: mean probability and mean
// routed count per expert and their scaled dot product (gate.cuh:763-773). Every sum has a fixed
// order, so the loss does not depend on timing.
__device__ __forceinline__ void gate_loss_finalize(const LayerParams& p) {
    const uint32_t lane = threadIdx.x & 63, E = p.E;
    const float inv_s = 1.0f / float(p.S);
    float dot = 0.f;
    for (uint32_t e0 = 0; e0 < E; e0 += kWave) {
        const uint32_t e = e0 + lane;
        float prod = 0.f;
        if (e < E) {
            float total = 0.f;
            for (uint32_t r0 = 0; r0 < p.n_super; r0 += 16) {
                float v[16];
#pragma unroll
                for (uint32_t u = 0; u < 16; ++u)
                    v[u] = load_coherent(p.super_prob + size_t(r0 + u < p.n_super ? r0 + u : p.n_super - 1) * E + e);
#pragma unroll
                for (uint32_t u = 0; u < 16; ++u) total += r0 + u < p.n_super ? v[u] : 0.f;
            }
            const float mean_prob = total * inv_s;
            const float mean_count = float(load_coherent(p.expert_count + e)) * inv_s;
            p.gate_loss[e] = mean_prob;
            p.gate_loss[E + e] = mean_count;
            prod = mean_prob * mean_count;
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) prod += __shfl_xor(prod, off);
        dot += prod;
    }
    if (lane == 0) p.gate_loss[2 * E] = dot / float(E);
}

}  // namespace kleos_amd
