// Weighted combine: out[t] = sum over the kept experts of t of  Element(p_e) * Element(y_e * (1 / den_t)).
//
// Replaces processor::combine (csrc/include/kleos/os/processor/processor.cuh:44-205). The
// reference scatters each expert tile into the output with Element atomicAdd, in arrival order,
// onto a buffer zeroed at the start of the launch (moe.cuh:43-48). Here each token's row is
// gathered from the (at most k) expert rows that hold its results and summed in fp32 in selection
// order, which is deterministic, needs no zero fill and writes every output row exactly once
// (a token dropped by all its experts gets a zero row). With k == 1 the expert row is copied
// unscaled, as the reference does (processor.cuh:170-203).
#pragma once
#include "device_common.hpp"

namespace kleos_amd {

// One token per wavefront at a time; each lane handles 16-byte chunks of the row. A wavefront walks
// the tokens first, first + stride, ... and keeps two things in flight while it sums a token: all
// the expert rows of CH column chunks of that token, and the routing entries of its next token.
// Everything it reads was written by other workgroups of the same launch (routing by the gate and
// slot phases, y by the down-projection), hence the device-coherent loads; each y row is read
// exactly once, so nothing is lost by not serving it from the L2.
template <int KMAX>
struct CombineRoute {
    int32_t slot[KMAX];
    int32_t expert[KMAX];
    float prob[KMAX];
    float den;
};

template <int KMAX>
__device__ __forceinline__ CombineRoute<KMAX> combine_route(const LayerParams& p, uint32_t token) {
    CombineRoute<KMAX> r;
    r.den = load_coherent(p.combine_den + token);
#pragma unroll
    for (int i = 0; i < KMAX; ++i) {
        r.slot[i] = -1; r.expert[i] = 0; r.prob[i] = 0.f;
        if (uint32_t(i) < p.k) {
            r.slot[i] = load_coherent(p.topk_slot + size_t(token) * p.k + i);
            r.expert[i] = load_coherent(p.topk_expert + size_t(token) * p.k + i);
            r.prob[i] = load_coherent(p.topk_prob + size_t(token) * p.k + i);
        }
    }
    return r;
}

template <typename T, int KMAX, int CH>
__device__ __forceinline__ void combine_tokens_inline(const LayerParams& p, uint32_t first, uint32_t stride) {
    constexpr int kPer = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    const uint32_t H = p.H, k = p.k;
    const T* y = static_cast<const T*>(p.y);
    const uint32_t col_stride = kWave * kPer;
    // byte offset of column `col` inside a row of y (a lane's 16 bytes never straddle two pieces)
    auto row_offset = [&](uint32_t col) {
        if constexpr (sizeof(T) == 2) return uint32_t((size_t(col / kOutPiece) * p.cap_rows * kOutPiece + col % kOutPiece) * sizeof(T));
        else return uint32_t(col * sizeof(T));
    };

    if (first >= p.S) return;
    CombineRoute<KMAX> cur = combine_route<KMAX>(p, first);
    for (uint32_t token = first; token < p.S; token += stride) {
        CombineRoute<KMAX> nxt = cur;
        if (token + stride < p.S) nxt = combine_route<KMAX>(p, token + stride);
        // y / den as y * (1 / den): the reference divides with __fdividef (processor.cuh:135), an
        // approximate division, and a full IEEE division per element made this phase instruction-bound
        const float inv_den = __builtin_amdgcn_rcpf(cur.den);
        coherent_rows_t rows[KMAX];
        float scale[KMAX];
        bool on[KMAX];
#pragma unroll
        for (int r = 0; r < KMAX; ++r) {
            on[r] = cur.slot[r] >= 0;   // the same in every lane: a wavefront works on one token
            // (indices clamped to their tables: no value they could hold leaves the y buffer)
            const uint32_t e = uint32_t(cur.expert[r]) < p.E ? uint32_t(cur.expert[r]) : p.E - 1;
            const uint32_t sl = uint32_t(cur.slot[r]) < p.cap_rows ? uint32_t(cur.slot[r]) : p.cap_rows - 1;
            rows[r] = coherent_rows(y + (on[r] ? y_offset(e, sl, 0, p.cap_rows, H, sizeof(T)) : 0));
            scale[r] = elem_to_float(float_to_elem<T>(cur.prob[r]));
        }
        T* out = static_cast<T*>(p.moe_out) + size_t(token) * H;
        for (uint32_t c0 = lane * kPer; c0 < H; c0 += CH * col_stride) {
            u32x4 v[CH][KMAX];
#pragma unroll
            for (int c = 0; c < CH; ++c)
#pragma unroll
                for (int r = 0; r < KMAX; ++r)
                    if (on[r] && c0 + c * col_stride < H) v[c][r] = load16_coherent(rows[r], row_offset(c0 + c * col_stride));
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                if (c0 + c * col_stride >= H) break;
                // Element(gateOut[t, e]) * Element(fp32(y) * (1 / den)), summed in fp32 in selection order
                // (processor.cuh:117,135,146); with k == 1 the row is copied unscaled
                // (processor.cuh:170-203).
                float acc[kPer];
#pragma unroll
                for (int j = 0; j < kPer; ++j) acc[j] = 0.f;
#pragma unroll
                for (int r = 0; r < KMAX; ++r) {
                    if (!on[r]) continue;
                    T vals[kPer];
                    __builtin_memcpy(vals, &v[c][r], 16);
#pragma unroll
                    for (int j = 0; j < kPer; ++j) {
                        if (k == 1) acc[j] = elem_to_float(vals[j]);
                        else acc[j] = fmaf(scale[r], elem_to_float(float_to_elem<T>(elem_to_float(vals[j]) * inv_den)), acc[j]);
                    }
                }
                T o[kPer];
#pragma unroll
                for (int j = 0; j < kPer; ++j) o[j] = float_to_elem<T>(acc[j]);
                u32x4 raw;
                __builtin_memcpy(&raw, o, 16);
                store16(out + c0 + c * col_stride, raw);
            }
        }
        cur = nxt;
    }
}

// Any k: the routing entries are re-read for every column chunk.
template <typename T>
__device__ __forceinline__ void combine_tokens_generic(const LayerParams& p, uint32_t first, uint32_t stride) {
    constexpr int kPer = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    const uint32_t H = p.H, k = p.k;
    const T* y = static_cast<const T*>(p.y);
    for (uint32_t token = first; token < p.S; token += stride) {
        const float inv_den = __builtin_amdgcn_rcpf(load_coherent(p.combine_den + token));
        T* out = static_cast<T*>(p.moe_out) + size_t(token) * H;
        for (uint32_t c0 = lane * kPer; c0 < H; c0 += kWave * kPer) {
            float acc[kPer];
#pragma unroll
            for (int j = 0; j < kPer; ++j) acc[j] = 0.f;
            for (uint32_t r = 0; r < k; ++r) {
                const int32_t slot = load_coherent(p.topk_slot + size_t(token) * k + r);
                if (slot < 0) continue;
                uint32_t e = uint32_t(load_coherent(p.topk_expert + size_t(token) * k + r));
                if (e >= p.E || uint32_t(slot) >= p.cap_rows) continue;
                const float scale = elem_to_float(float_to_elem<T>(load_coherent(p.topk_prob + size_t(token) * k + r)));
                const u32x4 raw = load16_coherent(coherent_rows(y + y_offset(e, uint32_t(slot), 0, p.cap_rows, H, sizeof(T))),
                                                  uint32_t((y_offset(0, 0, c0, p.cap_rows, H, sizeof(T))) * sizeof(T)));
                T vals[kPer];
                __builtin_memcpy(vals, &raw, 16);
#pragma unroll
                for (int j = 0; j < kPer; ++j)
                    acc[j] = fmaf(scale, elem_to_float(float_to_elem<T>(elem_to_float(vals[j]) * inv_den)), acc[j]);
            }
            T o[kPer];
#pragma unroll
            for (int j = 0; j < kPer; ++j) o[j] = float_to_elem<T>(acc[j]);
            u32x4 raw;
            __builtin_memcpy(&raw, o, 16);
            store16(out + c0, raw);
        }
    }
}

// Tokens first, first + stride, ... of the calling wavefront.
template <typename T>
__device__ __forceinline__ void combine_tokens(const LayerParams& p, uint32_t first, uint32_t stride) {
    if (p.k <= 2) combine_tokens_inline<T, 2, 4>(p, first, stride);
    else if (p.k <= 4) combine_tokens_inline<T, 4, 4>(p, first, stride);
    else if (p.k <= 8) combine_tokens_inline<T, 8, 2>(p, first, stride);
    else combine_tokens_generic<T>(p, first, stride);
}

}  // namespace kleos_amd
