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
// bf16, matrix cores. WAVES_M x WAVES_N wavefronts over a BM x BN tile (two wavefronts per SIMD with
// eight of them, so that one's LDS waits hide behind the other's matrix instructions).
//
// K is walked in slices of 64 through a ring of LDS stages that the wavefronts fill with direct
// global->LDS loads (global_load_lds_dwordx4: each lane names a 16-byte global source, the 64 lanes
// of the instruction land in 1 KB of consecutive LDS). The loads of the next slice are issued
// before the current slice is multiplied, so they have a whole slice of matrix work to arrive and
// never occupy a vector register. A slice holds 128 bytes of every row, i.e. whole cache lines:
// narrower slices make consecutive loads hit lines whose miss is still pending, which stalls the
// L1. Rows of A are gathered through the slot->token table by giving each lane its token's row
// address.
//
// LDS layout of a stage: rows of 128 bytes (64 bf16), 16-byte chunk c of row r stored at chunk
// position c ^ swz(r). The LDS of gfx950 has 64 banks of 4 bytes (two tile rows per bank row) and
// serves a 16-byte access of 16 lanes per clock; with this swizzle any 16 consecutive rows read at
// one chunk index cover all 64 banks. Because the LDS destination of a direct load is fixed by the
// lane number, the swizzle is applied on the global side: lane (r, p) fetches chunk p ^ swz(r) of
// its row.
//
// The weight rows feed the matrix core's row operand and the activation rows its column operand,
// i.e. the core computes C^T: a lane then owns 4 consecutive output columns of one output row.
// ------------------------------------------------------------------------------------------------
constexpr int kGemmBK = 64;
constexpr int kGemmStages = 2;
#ifdef KLEOS_TRACE
__device__ unsigned long long* g_trace = nullptr;   // diagnostic build only
#endif

__device__ __forceinline__ int swz(int r) { return ((r >> 1) & 7) ^ ((r & 1) << 2); }

template <int BM, int BN>
constexpr int gemm_bf16_smem_bytes() { return kGemmStages * (BM + BN) * kGemmBK * 2; }

typedef const __attribute__((address_space(1))) void* global_cptr;
typedef __attribute__((address_space(3))) void* lds_ptr;

// Waits until at most N of this wavefront's vector-memory operations are outstanding.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64);
    // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// A_AUX: cache-policy bits of the loads of A (0 = default, 1 = sc0: do not trust this CU's L1, for
// rows another workgroup of the same launch has just written).
template <int ACT, int BM, int BN, int WAVES_M, int WAVES_N, int A_AUX>
__device__ __forceinline__ void gemm_tile_bf16(
    const bf16_t* __restrict__ a_base, const int32_t* __restrict__ a_row_index, uint32_t lda,
    uint32_t m_valid,
    const bf16_t* __restrict__ b_base, uint32_t ldb, uint32_t n_valid,
    const bf16_t* __restrict__ bias, bf16_t* __restrict__ c_base, uint32_t ldc, uint32_t K,
    char* smem) {
    constexpr int kGemmWaves = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;   // wavefront tile
    constexpr int TM = WM / 32, TN = WN / 32;             // 32x32 matrix-core tiles per wavefront
    static_assert(WM % 32 == 0 && WN % 32 == 0);
    constexpr int kRowBytes = kGemmBK * 2;                // 128
    constexpr int kABytes = BM * kRowBytes, kBBytes = BN * kRowBytes;
    constexpr int kStage = kABytes + kBBytes;
    // one direct load covers 8 rows (1 KB); each wavefront issues LA + LB of them per stage
    static_assert(BM % (8 * kGemmWaves) == 0 && BN % (8 * kGemmWaves) == 0);
    constexpr int LA = BM / (8 * kGemmWaves), LB = BN / (8 * kGemmWaves);
    constexpr int kLoadsPerStage = LA + LB;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // Global source of this lane for each of its direct loads. Rows past the valid range re-read
    // the last valid row: their products land in accumulator rows / columns that are never stored.
    const int ld_r = lane >> 3, ld_p = lane & 7;
    const bf16_t* pa[LA];
    const bf16_t* pb[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = 8 * (wave + kGemmWaves * i) + ld_r;
        uint32_t r = row < int(m_valid) ? row : m_valid - 1;
        const size_t src = a_row_index ? size_t(a_row_index[r]) : size_t(r);
        pa[i] = a_base + src * lda + ((ld_p ^ swz(row)) << 3);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = 8 * (wave + kGemmWaves * i) + ld_r;
        uint32_t r = row < int(n_valid) ? row : n_valid - 1;
        pb[i] = b_base + size_t(r) * ldb + ((ld_p ^ swz(row)) << 3);
    }
    // part `part` of `parts` of the direct loads that bring slice kt into `stage`
    auto issue_part = [&](uint32_t kt, int stage, int part, int parts) {
        char* sa = smem + stage * kStage;
        char* sb = sa + kABytes;
        const uint32_t k0 = kt * kGemmBK;
#pragma unroll
        for (int i = 0; i < LA; ++i)
            if (i * parts / LA == part)
                __builtin_amdgcn_global_load_lds((global_cptr)(pa[i] + k0),
                                                 (lds_ptr)(sa + 1024 * (wave + kGemmWaves * i)), 16, 0, A_AUX);
#pragma unroll
        for (int i = 0; i < LB; ++i)
            if (i * parts / LB == part)
                __builtin_amdgcn_global_load_lds((global_cptr)(pb[i] + k0),
                                                 (lds_ptr)(sb + 1024 * (wave + kGemmWaves * i)), 16, 0, 0);
    };
    auto issue = [&](uint32_t kt, int stage) { issue_part(kt, stage, 0, 1); };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int ni = 0; ni < TN; ++ni)
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ni][mi][v] = 0.f;

    const uint32_t k_tiles = K / kGemmBK;
    // prologue: the first kGemmStages - 1 slices in flight
#pragma unroll
    for (int st = 0; st < kGemmStages - 1; ++st)
        if (uint32_t(st) < k_tiles) issue(st, st);

    const int fr_row = lane & 31, fr_half = lane >> 5;
    constexpr int kSteps = kGemmBK / 16;   // matrix instructions consume 16 values of K
    // fragment byte offsets inside a stage for every K step of a slice
    int off_w[TN][kSteps], off_x[TM][kSteps];
#pragma unroll
    for (int ni = 0; ni < TN; ++ni) {
        const int r = wn * WN + ni * 32 + fr_row;
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) off_w[ni][ks] = kABytes + r * kRowBytes + (((ks * 2 + fr_half) ^ swz(r)) << 4);
    }
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) {
        const int r = wm * WM + mi * 32 + fr_row;
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) off_x[mi][ks] = r * kRowBytes + (((ks * 2 + fr_half) ^ swz(r)) << 4);
    }

#ifdef KLEOS_TRACE
    unsigned long long* trc = (blockIdx.x == KLEOS_TRACE && lane == 0 && g_trace) ? g_trace + wave * 256 : nullptr;
#define KTR(i) if (trc && kt < 32) trc[kt * 6 + (i)] = __builtin_readcyclecounter()
#else
#define KTR(i)
#endif
    for (uint32_t kt = 0; kt < k_tiles; ++kt) {
        KTR(0);
        // This wavefront's loads of slice kt have landed once only those of the later slices in
        // flight (kGemmStages - 2 of them, fewer at the end) are outstanding.
        if constexpr (kGemmStages == 2) {
            wait_vmcnt<0>();
        } else {
            static_assert(kGemmStages == 2 || kGemmStages == 3 || kGemmStages == 4);
            const uint32_t later = k_tiles - 1 - kt;   // slices after kt that exist
            if (later >= uint32_t(kGemmStages - 2)) wait_vmcnt<(kGemmStages - 2) * kLoadsPerStage>();
            else if (kGemmStages == 4 && later == 1) wait_vmcnt<kLoadsPerStage>();
            else wait_vmcnt<0>();
        }
        // every wavefront's share of slice kt is in LDS, and everyone has finished reading slice
        // kt-1, whose stage the next loads overwrite
        KTR(1);
        asm volatile("s_barrier" ::: "memory");
        KTR(2);
        // The loads of the next slice are spread over the K steps of this one: issued in one
        // burst they queue up in the texture addresser and hold the wavefront (and with it its
        // matrix instructions) until the last one is accepted.
        const bool more = kt + kGemmStages - 1 < k_tiles;
        const uint32_t next_kt = kt + kGemmStages - 1;
        const int next_stage = next_kt % kGemmStages;
        KTR(3);
        const char* st = smem + (kt % kGemmStages) * kStage;
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
            bf16x8 fw[TN], fx[TM];
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) fw[ni] = __builtin_bit_cast(bf16x8, load16(st + off_w[ni][ks]));
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) fx[mi] = __builtin_bit_cast(bf16x8, load16(st + off_x[mi][ks]));
            if (more) issue_part(next_kt, next_stage, ks, kSteps);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ni = 0; ni < TN; ++ni)
#pragma unroll
                for (int mi = 0; mi < TM; ++mi)
                    acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[ni], fx[mi], acc[ni][mi], 0, 0, 0);
        }
        KTR(4);
    }
    // all wavefronts are done with the ring: each now reuses its own 1/8 of it
    __syncthreads();

    // Epilogue. acc[ni][mi][v] is output column n = wn*WN + ni*32 + 8*(v/4) + 4*(lane/32) + v%4 of
    // output row m = wm*WM + mi*32 + lane%32: a lane owns 4 consecutive columns of 16 rows. Bias,
    // activation and the rounding to Element happen in registers; the wavefront then transposes its
    // WM x WN block through a private LDS region (rows of WN*2 bytes, 16-byte chunk c of row r at
    // position c ^ ((r >> 1) & 7)) so that the global stores are 16 bytes per lane and cover whole
    // 128-byte lines of the output rows.
    static_assert(WN % 64 == 0, "epilogue staging works on 64-column (128-byte) panels");
    static_assert(WM * WN * 2 * kGemmWaves <= gemm_bf16_smem_bytes<BM, BN>());
    char* stg_wave = smem + wave * (WM * WN * 2);
#pragma unroll
    for (int pn = 0; pn < WN / 64; ++pn) {                  // 64-column panel of the wavefront tile
        char* stg = stg_wave + pn * (WM * 128);
#pragma unroll
        for (int nl = 0; nl < 2; ++nl) {
            const int ni = pn * 2 + nl;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t n = wn * WN + ni * 32 + 8 * q + 4 * fr_half;
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (n < n_valid) {
                    const bf16x4 b4 = *reinterpret_cast<const bf16x4*>(bias + n);
#pragma unroll
                    for (int j = 0; j < 4; ++j) bv[j] = float(b4[j]);
                }
#pragma unroll
                for (int mi = 0; mi < TM; ++mi) {
                    const int r = mi * 32 + fr_row;
                    bf16x4 o;
#pragma unroll
                    for (int j = 0; j < 4; ++j) o[j] = static_cast<bf16_t>(activate<ACT>(acc[ni][mi][4 * q + j] + bv[j]));
                    *reinterpret_cast<bf16x4*>(stg + r * 128 + (((nl * 4 + q) ^ ((r >> 1) & 7)) << 4) + fr_half * 8) = o;
                }
            }
        }
        // same wavefront wrote and reads the region: LDS operations of one wavefront complete in order
#pragma unroll
        for (int it = 0; it < WM * 8 / kWave; ++it) {
            const int id = it * kWave + lane;
            const int r = id >> 3, c = id & 7;
            const u32x4 v = load16(stg + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
            const uint32_t m = wm * WM + r, n = wn * WN + pn * 64 + c * 8;
            if (m < m_valid && n < n_valid) store16(c_base + size_t(m) * ldc + n, v);
        }
    }
    // the caller may start the next tile's loads into the ring right away
    __syncthreads();
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
