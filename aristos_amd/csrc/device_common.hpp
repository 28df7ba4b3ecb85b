// Small device-side vocabulary shared by the kernels: vector types, Element conversions,
// matrix-core wrappers, scoped atomics.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "layer.hpp"

namespace kleos_amd {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// tf32 (torch_dtype 1, the reference's cute::tfloat32_t, csrc/include/kleos/types.cuh:128-131): an
// Element stored in 32 bits of which the matrix cores of the reference's hardware read the sign,
// the exponent and the upper 10 mantissa bits. CDNA4 has no tf32 matrix instruction: the fp32
// matrix instructions run on operands whose lower 13 mantissa bits are cleared (products of two
// such values are exact in fp32, as they are in a tf32 tensor core), and every Element the layer
// produces is rounded to 10 mantissa bits, ties to even, with the lower bits cleared
// (cutlass::NumericConverter<tfloat32_t, float> rounds the same way and leaves the lower bits
// undefined).
struct tf32_t { float v; };
__device__ __forceinline__ float tf32_operand(float v) {
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) & 0xffffe000u);
}
__device__ __forceinline__ float tf32_round(float v) {
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7f800000u) != 0x7f800000u) u += 0x0fffu + ((u >> 13) & 1u);   // infinities and NaNs keep their bits
    return __builtin_bit_cast(float, u & 0xffffe000u);
}

__device__ __forceinline__ float elem_to_float(bf16_t v) { return static_cast<float>(v); }
__device__ __forceinline__ float elem_to_float(tf32_t v) { return v.v; }   // as stored (a bias, a gate output)
__device__ __forceinline__ float elem_to_float(f16_t v) { return static_cast<float>(v); }
__device__ __forceinline__ float elem_to_float(float v) { return v; }

// fp32 -> Element, round to nearest even (cutlass::NumericConverter in the reference).
template <typename T>
__device__ __forceinline__ T float_to_elem(float v);
template <>
__device__ __forceinline__ float float_to_elem<float>(float v) { return v; }
template <>
__device__ __forceinline__ tf32_t float_to_elem<tf32_t>(float v) { return tf32_t{tf32_round(v)}; }
template <>
__device__ __forceinline__ bf16_t float_to_elem<bf16_t>(float v) { return static_cast<bf16_t>(v); }
template <>
__device__ __forceinline__ f16_t float_to_elem<f16_t>(float v) { return static_cast<f16_t>(v); }

// The two 16-bit Elements share every kernel; what differs is the vector types and the matrix
// instructions.
template <typename E> struct Elem16;
template <> struct Elem16<bf16_t> {
    typedef bf16x8 vec8;
    typedef bf16x4 vec4;
    static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Elem16<f16_t> {
    typedef f16x8 vec8;
    typedef f16x4 vec4;
    static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void store16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// Activations of the reference (types.cuh:151-159): 0 = ReLU<float>, 1 = erf GELU<float>.
template <int ACT>
__device__ __forceinline__ float activate(float v) {
    if constexpr (ACT == 0) return v > 0.0f ? v : 0.0f;
    else if constexpr (ACT == 1) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    else return v;
}

// One matrix-core step on 16 bytes of K per lane from each operand, 16x16 output.
//   a: lane l holds row  (l % 16) of the 16-row operand, K-chunk (l / 16)
//   b: lane l holds col  (l % 16) of the 16-col operand, K-chunk (l / 16)
//   acc[v]: element (row 4*(l/16)+v, col l%16)
// For bf16 one instruction consumes 32 values of K; for fp32 four instructions consume 16.
__device__ __forceinline__ f32x4 mma16_step(u32x4 a, u32x4 b, f32x4 acc, bf16_t) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma16_step(u32x4 a, u32x4 b, f32x4 acc, f16_t) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma16_step(u32x4 a, u32x4 b, f32x4 acc, float) {
    f32x4 fa = __builtin_bit_cast(f32x4, a), fb = __builtin_bit_cast(f32x4, b);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[0], fb[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[1], fb[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[2], fb[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[3], fb[3], acc, 0, 0, 0);
    return acc;
}

// tf32: the same fp32 instructions on operands cut to their upper 10 mantissa bits.
__device__ __forceinline__ f32x4 mma16_step(u32x4 a, u32x4 b, f32x4 acc, tf32_t) {
    const u32x4 mask{0xffffe000u, 0xffffe000u, 0xffffe000u, 0xffffe000u};
    return mma16_step(a & mask, b & mask, acc, float{});
}

// The value another lane of the same row of 16 lanes holds, by the lane selects of the vector ALU
// (no trip through the LDS crossbar as a general shuffle takes). STEP 0: lane ^ 1, 1: lane ^ 2,
// 2: lane ^ 7, 3: lane ^ 15. Steps 0..3 in this order are an all-reduce over the 16 lanes for any
// operation whose result does not depend on the order of its two operands: after steps 0 and 1 the
// four lanes of a quad agree, so the mirrored lane of step 2 (in the other quad of the same eight)
// holds what lane ^ 4 holds, and likewise lane ^ 15 what lane ^ 8 holds in step 3.
template <int STEP>
__device__ __forceinline__ uint32_t row16_peer(uint32_t v) {
    static_assert(STEP >= 0 && STEP < 4);
    constexpr int kCtrl = STEP == 0 ? 0xB1      // quad_perm [1, 0, 3, 2]
                        : STEP == 1 ? 0x4E      // quad_perm [2, 3, 0, 1]
                        : STEP == 2 ? 0x141     // row_half_mirror
                                    : 0x140;    // row_mirror
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), kCtrl, 0xF, 0xF, false));
}
template <int STEP>
__device__ __forceinline__ float row16_peer(float v) {
    return __builtin_bit_cast(float, row16_peer<STEP>(__builtin_bit_cast(uint32_t, v)));
}
// op(a, b) == op(b, a) bit for bit (max, +): every lane of the row ends with the same value, combined
// in the order of a xor butterfly over 1, 2, 4, 8.
template <typename Op>
__device__ __forceinline__ float row16_allreduce(float v, Op op) {
    v = op(v, row16_peer<0>(v));
    v = op(v, row16_peer<1>(v));
    v = op(v, row16_peer<2>(v));
    v = op(v, row16_peer<3>(v));
    return v;
}

// Waits until at most N of this wavefront's vector-memory operations (loads and stores alike) are
// outstanding.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64);
    // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// Device-scope (agent) atomics: the scheduler counters are shared by workgroups on different
// XCDs, whose L2 caches are not coherent with each other for ordinary loads and stores.
__device__ __forceinline__ uint32_t atomic_add_agent(uint32_t* p, uint32_t v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t atomic_load_relaxed(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void atomic_store_relaxed(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Data that crosses workgroups inside one launch. The eight L2 caches of the device are not
// coherent with each other: a plain store may stay in the writer's L2, and a line read in an
// earlier phase or launch may still sit in the reader's. Writing such data back with a
// device-scope release and dropping stale lines with a device-scope acquire walks a whole L2 each
// time (about 2 us per release at a grid-wide barrier, tens of microseconds of refetching per
// acquire), so the tables and rows that cross workgroups are instead written and read with the
// agent scope (sc1) on the instructions themselves:
//   * store_through / store16_through / the sc1 buffer stores of the GEMM epilogue write through
//     the L2 to memory; once the wavefront's vmcnt has drained they are visible device-wide, which
//     is all a grid-wide barrier or a readiness counter has to wait for;
//   * load_coherent / load16_coherent are not served from a stale line.
template <typename V, typename U>
__device__ __forceinline__ void store_through(V* p, U v) {
    static_assert(sizeof(V) == 4 || sizeof(V) == 8);
    __hip_atomic_store(p, static_cast<V>(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes at a per-lane address (16-byte aligned).
__device__ __forceinline__ void store16_through(void* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
template <typename V>
__device__ __forceinline__ V load_coherent(const V* p) {
    static_assert(sizeof(V) == 4 || sizeof(V) == 8);
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte variant: buffer loads take the cache policy as an operand. `rows` describes memory that
// starts at a wavefront-uniform address; `byte_offset` may differ per lane.
typedef __amdgpu_buffer_rsrc_t coherent_rows_t;
__device__ __forceinline__ coherent_rows_t coherent_rows(const void* uniform_base) {
    const uint64_t a = reinterpret_cast<uint64_t>(uniform_base);
    // readfirstlane returns a signed int: both halves go through uint32_t before they are widened,
    // or a low half with its top bit set would smear ones over the high half
    const uint32_t lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(a))));
    const uint32_t hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(a >> 32))));
    const uint64_t u = (uint64_t(hi) << 32) | uint64_t(lo);
    // raw buffer: stride 0, 2 GiB window, 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(u), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ u32x4 load16_coherent(coherent_rows_t rows, uint32_t byte_offset) {
    constexpr int kAgentScope = 16;   // sc1
    return __builtin_amdgcn_raw_buffer_load_b128(rows, int(byte_offset), 0, kAgentScope);
}

}  // namespace kleos_amd
