// Gate: logits GEMM fused with softmax, top-k and the per-tile expert histogram, then the
// token-order slot assignment with capacity drop.
//
// Replaces gate::FusedGate / gate::forward of the reference (csrc/include/kleos/moe/gate.cuh:
// 474-720, 729-789). Differences that matter:
//   * one wavefront quad of lanes owns a token, so softmax and top-k are register + cross-lane
//     shuffle work; the reference bounces the accumulator through shared memory to get one
//     thread per token (gate.cuh:560-572);
//   * every expert count up to 256 is handled inside one workgroup (the reference chains
//     64-expert blocks through global-memory mailboxes, gate.cuh:93-468);
//   * slots are assigned in token order from per-tile histograms and their prefix sums, which
//     makes dropping deterministic; the reference takes a tile's base slot from atomicAdd arrival
//     order (gate.cuh:699).
#pragma once
#include "device_common.hpp"

namespace kleos_amd {

template <typename T>
struct GateK {
    static constexpr int kElemsPer16B = 16 / sizeof(T);
    // K consumed by one mma16_step: each of the 4 lane groups brings 16 bytes
    static constexpr int kStepK = 4 * kElemsPer16B;
};

// LDS floats needed by gate_tile: three partial accumulators of 4*NG registers for 64 lanes.
template <int NG>
constexpr int gate_smem_floats() { return 3 * NG * 4 * kWave; }

// One 16-token tile of the gate, computed by a group of four wavefronts (256 threads): the four
// waves split the hidden dimension, wave 0 of the group reduces the partial sums in a fixed order
// and runs the epilogue. A workgroup of 256*G threads runs G groups side by side on different
// tiles; every thread of the workgroup must call the function (it contains workgroup barriers) and
// a group without a tile passes valid = false. `smem` is the group's private scratch of
// gate_smem_floats<NG>() floats; it may be reused after the call (which ends with a barrier).
template <typename T, int NG>
__device__ __forceinline__ void gate_tile(const LayerParams& p, uint32_t tile, bool valid, float* smem) {
    const int tid = threadIdx.x & 255;
    const int wave = tid >> 6, lane = tid & 63;
    const int col = lane & 15;       // token inside the tile / expert row inside a group
    const int chunk = lane >> 4;     // which 16-byte K chunk of a step this lane loads
    const uint32_t H = p.H, E = p.E;
    const uint32_t token = tile * kGateTileTokens + col;
    constexpr int kStepK = GateK<T>::kStepK;
    constexpr int kPer = GateK<T>::kElemsPer16B;

    const uint32_t steps = H / kStepK;
    const uint32_t s0 = (steps * wave) / 4, s1 = (steps * (wave + 1)) / 4;

    const T* xrow = static_cast<const T*>(p.x) + size_t(token) * H + chunk * kPer;
    const T* wrow = static_cast<const T*>(p.wg) + size_t(col) * H + chunk * kPer;

    f32x4 acc[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // logits^T tile: experts are the matrix-core rows, tokens its columns (gate.cuh:526-534).
    // The loads of U steps are issued together before their matrix instructions: the activation
    // rows stream from HBM once and this is what keeps enough of them in flight.
    constexpr int U = NG <= 4 ? 4 : (NG <= 8 ? 2 : 1);
    uint32_t s = valid ? s0 : s1;
    for (; s + U <= s1; s += U) {
        u32x4 b[U], a[U][NG];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t off = (s + u) * kStepK;
            b[u] = load16(xrow + off);
#pragma unroll
            for (int g = 0; g < NG; ++g) a[u][g] = load16(wrow + size_t(g) * 16 * H + off);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int g = 0; g < NG; ++g) acc[g] = mma16_step(a[u][g], b[u], acc[g], T{});
    }
    for (; s < s1; ++s) {
        const uint32_t off = s * kStepK;
        const u32x4 b = load16(xrow + off);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const u32x4 a = load16(wrow + size_t(g) * 16 * H + off);
            acc[g] = mma16_step(a, b, acc[g], T{});
        }
    }

    if (valid && wave > 0) {
        float* dst = smem + (wave - 1) * (NG * 4 * kWave);
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) dst[(g * 4 + v) * kWave + lane] = acc[g][v];
    }
    __syncthreads();
    if (valid && wave == 0) {
        // fixed summation order: wave 0 + wave 1 + wave 2 + wave 3
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            const float* src = smem + w * (NG * 4 * kWave);
#pragma unroll
            for (int g = 0; g < NG; ++g)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[g][v] += src[(g * 4 + v) * kWave + lane];
        }

        // This lane holds, for its token, experts e = 16 g + 4 chunk + v.
        const float kNegInf = -__builtin_inff();
        float lg[NG][4];
        float m = kNegInf;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 16 * g + 4 * chunk + v;
                // softmax domain = the E real experts only (gate.cuh:550)
                lg[g][v] = e < E ? acc[g][v] : kNegInf;
                if (e < E) p.logits[size_t(token) * E + e] = acc[g][v];
                m = fmaxf(m, lg[g][v]);
            }
        m = fmaxf(m, __shfl_xor(m, 16));
        m = fmaxf(m, __shfl_xor(m, 32));
        float d = 0.f;
        float pr[NG][4];
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                pr[g][v] = __expf(lg[g][v] - m);   // exp(-inf) = 0 for padded experts
                d += pr[g][v];
            }
        d += __shfl_xor(d, 16);
        d += __shfl_xor(d, 32);
        const float inv_d = 1.0f / d;
        T* grow = static_cast<T*>(p.gate_out) + size_t(token) * p.PX;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 16 * g + 4 * chunk + v;
                pr[g][v] *= inv_d;
                // gateOut[t, e] = Element(p) (gate.cuh:590-605); padded columns are zero
                if (e < p.PX) grow[e] = float_to_elem<T>(e < E ? pr[g][v] : 0.f);
            }
        for (uint32_t e = 16 * NG + 4 * chunk; e < p.PX; e += 16) {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (e + v < p.PX) grow[e + v] = float_to_elem<T>(0.f);
        }

        // top-k: k rounds of arg-max, equal values go to the lower expert index (gate.cuh:654-670).
        int sel_round[NG][4];
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) sel_round[g][v] = -1;
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
                    if (e < E && sel_round[g][v] < 0 && (bi == kNone || lg[g][v] > best)) {
                        best = lg[g][v];
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
                        sel_round[g][v] = int(r);
                        pv = pr[g][v];
                    }
                }
            // exactly one of the four lanes of this token holds the winner; the others add 0
            pv += __shfl_xor(pv, 16);
            pv += __shfl_xor(pv, 32);
            den += pv;   // mCw, accumulated in selection order (gate.cuh:669)
            if (chunk == 0) {
                p.topk_expert[size_t(token) * p.k + r] = int32_t(bi);
                p.topk_prob[size_t(token) * p.k + r] = pv;
            }
        }
        if (chunk == 0) p.combine_den[token] = den;

        // Histogram of the tile and each token's rank inside it (gate.cuh:678-696).
        uint32_t* super = p.super_count + size_t(p.epoch & 1u) * p.n_super * E +
                          size_t(tile / kSuperTiles) * E;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = 16 * g + 4 * chunk + v;
                const bool sel = sel_round[g][v] >= 0;
                const unsigned long long mask = __ballot(sel);
                const uint32_t sub = uint32_t(mask >> (16 * chunk)) & 0xffffu;
                if (sel)
                    p.topk_slot[size_t(token) * p.k + sel_round[g][v]] =
                        int32_t(__popc(sub & ((1u << col) - 1u)));
                if (col == 0 && e < E) {
                    const uint32_t cnt = __popc(sub);
                    p.tile_count[size_t(tile) * E + e] = cnt;
                    if (cnt) atomic_add_agent(super + e, cnt);
                }
            }
    }
    __syncthreads();
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
            // total routed per expert, dropped tokens included (the reference's eC, gate.cuh:699)
            if (tile + 1 == p.n_gate_tiles)
                p.expert_count[e] = acc + load_coherent(p.tile_count + size_t(tile) * E + e);
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
            p.topk_slot[idx] = keep ? int32_t(slot) : -1;
            if (keep) p.slot_token[size_t(e) * p.cap_rows + slot] = int32_t(token);
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

}  // namespace kleos_amd
