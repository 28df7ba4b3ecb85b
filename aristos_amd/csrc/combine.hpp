// Weighted combine: out[t] = sum over the kept experts of t of  Element(p_e) * Element(y_e / den_t).
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

// One token per wavefront; each lane handles 16-byte chunks of the row. The routing of the token
// (at most kCombineInline experts on the fast path) is read once, then the expert rows of two
// column chunks are requested together so that a wavefront keeps 2k loads in flight.
constexpr int kCombineInline = 8;

template <typename T>
__device__ __forceinline__ void combine_token(const LayerParams& p, uint32_t token) {
    constexpr int kPer = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    const uint32_t H = p.H, k = p.k;
    const T* y = static_cast<const T*>(p.y);
    T* out = static_cast<T*>(p.moe_out) + size_t(token) * H;
    const float den = p.combine_den[token];
    const uint32_t stride = kWave * kPer;

    // Element(gateOut[t, e]) * Element(fp32(y) / den), summed in fp32 in selection order
    // (processor.cuh:117,135,146); with k == 1 the row is copied unscaled (processor.cuh:170-203).
    auto accumulate = [&](float (&accv)[kPer], const u32x4& raw, float scale) {
        T vals[kPer];
        __builtin_memcpy(vals, &raw, 16);
        if (k == 1) {
#pragma unroll
            for (int j = 0; j < kPer; ++j) accv[j] = elem_to_float(vals[j]);
        } else {
#pragma unroll
            for (int j = 0; j < kPer; ++j)
                accv[j] = fmaf(scale, elem_to_float(float_to_elem<T>(elem_to_float(vals[j]) / den)), accv[j]);
        }
    };
    auto store_row = [&](uint32_t c0, const float (&accv)[kPer]) {
        T o[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) o[j] = float_to_elem<T>(accv[j]);
        u32x4 raw;
        __builtin_memcpy(&raw, o, 16);
        store16(out + c0, raw);
    };

    if (k <= uint32_t(kCombineInline)) {
        const T* row[kCombineInline];
        float scale[kCombineInline];
#pragma unroll
        for (int r = 0; r < kCombineInline; ++r) {
            row[r] = nullptr;
            scale[r] = 0.f;
            if (uint32_t(r) < k) {
                const int32_t slot = p.topk_slot[size_t(token) * k + r];
                if (slot >= 0) {
                    const uint32_t e = uint32_t(p.topk_expert[size_t(token) * k + r]);
                    row[r] = y + (size_t(e) * p.cap_rows + uint32_t(slot)) * H;
                    scale[r] = elem_to_float(float_to_elem<T>(p.topk_prob[size_t(token) * k + r]));
                }
            }
        }
        uint32_t c0 = lane * kPer;
        for (; c0 + stride < H; c0 += 2 * stride) {
            u32x4 v0[kCombineInline], v1[kCombineInline];
#pragma unroll
            for (int r = 0; r < kCombineInline; ++r)
                if (row[r]) { v0[r] = load16(row[r] + c0); v1[r] = load16(row[r] + c0 + stride); }
            float a0[kPer], a1[kPer];
#pragma unroll
            for (int j = 0; j < kPer; ++j) { a0[j] = 0.f; a1[j] = 0.f; }
#pragma unroll
            for (int r = 0; r < kCombineInline; ++r)
                if (row[r]) { accumulate(a0, v0[r], scale[r]); accumulate(a1, v1[r], scale[r]); }
            store_row(c0, a0);
            store_row(c0 + stride, a1);
        }
        for (; c0 < H; c0 += stride) {
            float a0[kPer];
#pragma unroll
            for (int j = 0; j < kPer; ++j) a0[j] = 0.f;
#pragma unroll
            for (int r = 0; r < kCombineInline; ++r)
                if (row[r]) accumulate(a0, load16(row[r] + c0), scale[r]);
            store_row(c0, a0);
        }
        return;
    }

    for (uint32_t c0 = lane * kPer; c0 < H; c0 += stride) {
        float accv[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) accv[j] = 0.f;
        for (uint32_t r = 0; r < k; ++r) {
            const int32_t slot = p.topk_slot[size_t(token) * k + r];
            if (slot < 0) continue;
            const uint32_t e = uint32_t(p.topk_expert[size_t(token) * k + r]);
            const T* yrow = y + (size_t(e) * p.cap_rows + uint32_t(slot)) * H + c0;
            accumulate(accv, load16(yrow), elem_to_float(float_to_elem<T>(p.topk_prob[size_t(token) * k + r])));
        }
        store_row(c0, accv);
    }
}

}  // namespace kleos_amd
