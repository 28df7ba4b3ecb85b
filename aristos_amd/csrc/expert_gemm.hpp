// Expert projections: C[m, n] = act(sum_k A[m, k] * W[n, k] + bias[n]) on one output tile, with
// the rows of A optionally gathered through the slot->token table, so the dispatch of the
// reference (packet::dispatch row copy into a per-expert heap cell, csrc/include/kleos/os/
// packet.cuh:151-160) never materialises: the gather happens while the tile is staged into LDS.
//
// Replaces processor::fGET + BlockMM + FAA (csrc/include/kleos/os/processor/processor.cuh:358-489,
// gemm.cuh:22-107). Rounding points are the reference's: fp32 accumulate, fp32 bias add and
// activation, one round-to-nearest-even to Element on store (processor.cuh:475).
#pragma once
#include "device_common.hpp"

namespace kleos_amd {

// ------------------------------------------------------------------------------------------------
// bf16, matrix cores. 256 threads = 4 wavefronts arranged WAVES_M x WAVES_N over a BM x BN tile;
// K is walked in slices of 64 through a double-buffered, XOR-swizzled LDS tile (rows of 128 bytes,
// 16-byte chunk c of row r stored at chunk position c ^ (r & 7), which makes both the 16-byte
// stores of the staging pass and the ds_read_b128 fragment loads bank-conflict free).
//
// The weight rows feed the matrix core's row operand and the activation rows its column operand,
// i.e. the core computes C^T: a lane then owns 4 consecutive output columns of one output row and
// the epilogue packs them into one 8-byte store.
// ------------------------------------------------------------------------------------------------
constexpr int kGemmBK = 64;

template <int BM, int BN>
constexpr int gemm_bf16_smem_bytes() { return 2 * (BM + BN) * kGemmBK * 2; }

template <int ACT, int BM, int BN, int WAVES_M, int WAVES_N>
__device__ __forceinline__ void gemm_tile_bf16(
    const bf16_t* __restrict__ a_base, const int32_t* __restrict__ a_row_index, uint32_t lda,
    uint32_t m_valid,
    const bf16_t* __restrict__ b_base, uint32_t ldb, uint32_t n_valid,
    const bf16_t* __restrict__ bias, bf16_t* __restrict__ c_base, uint32_t ldc, uint32_t K,
    char* smem) {
    static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;   // wavefront tile
    constexpr int TM = WM / 32, TN = WN / 32;             // 32x32 matrix-core tiles per wavefront
    static_assert(WM % 32 == 0 && WN % 32 == 0 && BM % 32 == 0 && BN % 32 == 0);
    constexpr int PA = BM / 32, PB = BN / 32;             // staging passes (32 rows x 8 chunks each)
    constexpr int kABytes = BM * kGemmBK * 2, kBBytes = BN * kGemmBK * 2;
    constexpr int kStage = kABytes + kBBytes;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int ld_row = tid >> 3, ld_ch = tid & 7;

    // Source row pointers of this thread's staging chunks; nullptr rows are staged as zeros.
    const bf16_t* pa[PA];
    const bf16_t* pb[PB];
#pragma unroll
    for (int i = 0; i < PA; ++i) {
        const uint32_t r = ld_row + 32 * i;
        if (r < m_valid) {
            const size_t src = a_row_index ? size_t(a_row_index[r]) : size_t(r);
            pa[i] = a_base + src * lda + ld_ch * 8;
        } else {
            pa[i] = nullptr;
        }
    }
#pragma unroll
    for (int i = 0; i < PB; ++i) {
        const uint32_t r = ld_row + 32 * i;
        pb[i] = r < n_valid ? b_base + size_t(r) * ldb + ld_ch * 8 : nullptr;
    }
    const int st_off = ld_row * 128 + ((ld_ch ^ (ld_row & 7)) << 4);   // + 32*i rows = + 4096*i bytes

    f32x16 acc[TN][TM];
#pragma unroll
    for (int ni = 0; ni < TN; ++ni)
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ni][mi][v] = 0.f;

    u32x4 ra[PA], rb[PB];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < PA; ++i) ra[i] = pa[i] ? load16(pa[i] + k0) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < PB; ++i) rb[i] = pb[i] ? load16(pb[i] + k0) : u32x4{0u, 0u, 0u, 0u};
    };
    auto stage = [&](int buf) {
        char* sa = smem + buf * kStage;
        char* sb = sa + kABytes;
#pragma unroll
        for (int i = 0; i < PA; ++i) store16(sa + st_off + i * 4096, ra[i]);
#pragma unroll
        for (int i = 0; i < PB; ++i) store16(sb + st_off + i * 4096, rb[i]);
    };

    const uint32_t k_tiles = K / kGemmBK;
    fetch(0);
    stage(0);
    __syncthreads();

    const int fr_row = lane & 31, fr_half = lane >> 5;
    for (uint32_t kt = 0; kt < k_tiles; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < k_tiles) fetch((kt + 1) * kGemmBK);
        const char* sa = smem + buf * kStage;
        const char* sb = sa + kABytes;
#pragma unroll
        for (int ks = 0; ks < kGemmBK / 16; ++ks) {
            const int ch = ks * 2 + fr_half;
            bf16x8 fw[TN], fx[TM];
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
                const int r = wn * WN + ni * 32 + fr_row;
                fw[ni] = __builtin_bit_cast(bf16x8, load16(sb + r * 128 + ((ch ^ (r & 7)) << 4)));
            }
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) {
                const int r = wm * WM + mi * 32 + fr_row;
                fx[mi] = __builtin_bit_cast(bf16x8, load16(sa + r * 128 + ((ch ^ (r & 7)) << 4)));
            }
#pragma unroll
            for (int ni = 0; ni < TN; ++ni)
#pragma unroll
                for (int mi = 0; mi < TM; ++mi)
                    acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[ni], fx[mi], acc[ni][mi], 0, 0, 0);
        }
        if (kt + 1 < k_tiles) stage(buf ^ 1);
        __syncthreads();
    }

    // Epilogue. acc[ni][mi][v]: output column n = wn*WN + ni*32 + 8*(v/4) + 4*(lane/32) + v%4,
    // output row m = wm*WM + mi*32 + lane%32.
#pragma unroll
    for (int ni = 0; ni < TN; ++ni) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t n = wn * WN + ni * 32 + 8 * q + 4 * fr_half;
            if (n >= n_valid) continue;
            float bv[4];
            const bf16x4 b4 = *reinterpret_cast<const bf16x4*>(bias + n);
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = float(b4[j]);
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) {
                const uint32_t m = wm * WM + mi * 32 + fr_row;
                if (m >= m_valid) continue;
                bf16x4 o;
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = static_cast<bf16_t>(activate<ACT>(acc[ni][mi][4 * q + j] + bv[j]));
                *reinterpret_cast<bf16x4*>(c_base + size_t(m) * ldc + n) = o;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// fp32, vector ALU. 64 x 64 x 16 tile, 256 threads, 4 x 4 outputs per thread, K summed in
// ascending order. Serves the fp32 configuration, whose sizes are small.
// ------------------------------------------------------------------------------------------------
constexpr int kF32Tile = 64, kF32BK = 16, kF32Pad = 68;
constexpr int gemm_f32_smem_bytes() { return 2 * kF32BK * kF32Pad * 4; }

template <int ACT>
__device__ __forceinline__ void gemm_tile_f32(
    const float* __restrict__ a_base, const int32_t* __restrict__ a_row_index, uint32_t lda,
    uint32_t m_valid,
    const float* __restrict__ b_base, uint32_t ldb, uint32_t n_valid,
    const float* __restrict__ bias, float* __restrict__ c_base, uint32_t ldc, uint32_t K,
    char* smem) {
    float (*As)[kF32Pad] = reinterpret_cast<float (*)[kF32Pad]>(smem);
    float (*Bs)[kF32Pad] = reinterpret_cast<float (*)[kF32Pad]>(smem + kF32BK * kF32Pad * 4);
    const int tid = threadIdx.x;
    const int ld_row = tid >> 2, ld_kq = tid & 3;
    const int ty = tid >> 4, tx = tid & 15;

    const float* pa = nullptr;
    const float* pb = nullptr;
    if (uint32_t(ld_row) < m_valid) {
        const size_t src = a_row_index ? size_t(a_row_index[ld_row]) : size_t(ld_row);
        pa = a_base + src * lda + ld_kq * 4;
    }
    if (uint32_t(ld_row) < n_valid) pb = b_base + size_t(ld_row) * ldb + ld_kq * 4;

    float acc[4][4] = {};
    for (uint32_t k0 = 0; k0 < K; k0 += kF32BK) {
        const f32x4 va = pa ? *reinterpret_cast<const f32x4*>(pa + k0) : f32x4{0.f, 0.f, 0.f, 0.f};
        const f32x4 vb = pb ? *reinterpret_cast<const f32x4*>(pb + k0) : f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            As[ld_kq * 4 + j][ld_row] = va[j];
            Bs[ld_kq * 4 + j][ld_row] = vb[j];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kF32BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; b[i] = Bs[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t m = ty * 4 + i;
        if (m >= m_valid) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t n = tx * 4 + j;
            if (n < n_valid) c_base[size_t(m) * ldc + n] = activate<ACT>(acc[i][j] + bias[n]);
        }
    }
}

}  // namespace kleos_amd
