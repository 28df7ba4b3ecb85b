/*
 * moe_ref.c — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the single-GPU MoE-layer forward of Kleos/FlashDMoE. It exists so that the
 * HIP path can be checked against the reference's semantics; nothing in the shipped library links
 * or calls it. The reference itself (CUDA + NVSHMEM + CUTLASS, fetched over the network by its
 * CMake) cannot be built in this environment and holds no test vectors, so every function below is
 * pinned by independent checks in tests/ (an independent numpy/torch restatement, closed forms,
 * brute force), not by reference output.
 *
 * What each function follows (paths under the reference's csrc/include/kleos/):
 *   moe_ref_derive       types.cuh:471-507        PX, EC, pEC                       pinned: closed-form table
 *   moe_ref_gate_logits  moe/gate.cuh:526-534     logits = x * Wg^T, fp32 acc       pinned: torch fp64 matmul
 *   moe_ref_softmax      moe/gate.cuh:556-584     online max/denominator, E real    pinned: torch fp64 softmax,
 *                                                 experts only                              rows sum to 1
 *   moe_ref_topk         moe/gate.cuh:654-670     k rounds, strict '>' ascending e  pinned: stable-sort brute force,
 *                                                 => ties to the lower index;               crafted ties
 *                                                 combine_den = sum of selected p
 *   moe_ref_slots        moe/gate.cuh:678-718,    rank in token order, keep iff     pinned: O(S*k) brute force,
 *                        os/packet.cuh:85,112     slot < EC                                 permutation invariants
 *   expert FFN           os/processor/processor.cuh:706-741, gemm.cuh:22-31       pinned: torch fp64 matmul + relu/erf
 *                        h1 = Elem(act(x Wup^T + bup)); y = Elem(h1 Wdown^T + bdown)
 *   combine              os/processor/processor.cuh:110-168 (k>1), :170-203 (k=1) pinned: identity-expert, dense
 *                        out[t] += Elem(gateOut[t,e]) * Elem(y/combine_den)               mixture, k=1, all-dropped
 *                                                                                           closed forms
 *   zero-initialised output  moe/moe.cuh:43-48
 *   moe_ref_gate_loss    moe/gate.cuh:608-635 (mean probability per expert), :700-705 (mean    pinned: uniform logits give
 *                        routed count per expert), :763-773 (loss = sum of products / E)        k / E^2; both means sum to 1
 *                                                                                               and k; numpy restatement
 *
 * Deliberate, documented choices where the reference is schedule- or hardware-dependent:
 *   - top-k is selected on the fp32 LOGITS (order-equivalent to the probabilities the reference
 *     compares wherever exp() keeps distinct logits distinct; where it does not, the reference's
 *     answer depends on NVIDIA's ex2.approx and cannot be reproduced);
 *   - slots are handed out in token order (the reference's inter-tile order is atomicAdd arrival
 *     order, gate.cuh:699; token order is one of its legal outcomes and the one the task fixes);
 *   - the k>1 combine accumulates in Element in ascending expert index (the reference uses
 *     Element atomicAdd in arrival order, processor.cuh:157,165);
 *   - a k=1 token whose expert dropped it yields a zero row (the reference leaves the row
 *     unwritten).
 *   - tf32 (torch_dtype 1): the conversion is CUTLASS's (absent third-party code, restated; see
 *     moe_ref_round_tf32), pinned against an independent frexp/rint/ldexp rounding and crafted ties;
 *     that a tf32 tensor core ignores the lower 13 operand bits is the hardware's documented
 *     behaviour, which no file of the reference states: parity unpinned for that choice;
 *   Functions whose exact bits only a run of the reference could fix (fast-math exp/div ULPs,
 *   atomic order) are "parity unpinned" at the bit level and are compared within tolerance.
 */
#include "moe_ref.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ Element helpers */
uint16_t moe_ref_f32_to_bf16_bits(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest, ties to even */
    return (uint16_t)(u >> 16);
}
float moe_ref_bf16_bits_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float v;
    memcpy(&v, &u, 4);
    return v;
}
float moe_ref_round_bf16(float v) { return moe_ref_bf16_bits_to_f32(moe_ref_f32_to_bf16_bits(v)); }

/* IEEE binary16 by integer arithmetic: round to nearest, ties to even; overflow to infinity,
 * gradual underflow to subnormals (what cutlass::NumericConverter<half_t, float> does). */
uint16_t moe_ref_f32_to_f16_bits(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);          /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);         /* >= 65536 (and inf): infinity */
    if (a < 0x33000000u) return sign;                                /* < 2^-25: zero */
    const int exp = (int)(a >> 23) - 127;
    uint32_t mant = (a & 0x007fffffu) | 0x00800000u;                 /* 24-bit significand */
    int shift;                                                       /* bits dropped from it */
    uint32_t base;                                                   /* half bits before the mantissa is added */
    if (exp < -14) { shift = 13 + (-14 - exp); base = 0; }           /* subnormal half */
    else { shift = 13; base = (uint32_t)(exp + 15 - 1) << 10; }      /* implicit bit carries into the exponent */
    const uint32_t kept = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t h = base + kept;
    if (rem > half || (rem == half && (kept & 1u))) ++h;             /* may carry up to infinity: correct */
    return (uint16_t)(sign | h);
}
float moe_ref_f16_bits_to_f32(uint16_t b) {
    const uint32_t sign = (uint32_t)(b & 0x8000u) << 16;
    const uint32_t exp = (b >> 10) & 0x1fu, mant = b & 0x3ffu;
    uint32_t u;
    if (exp == 0x1fu) u = sign | 0x7f800000u | (mant << 13);
    else if (exp != 0) u = sign | ((exp + 112u) << 23) | (mant << 13);
    else if (mant == 0) u = sign;
    else {
        /* subnormal: value = mant * 2^-24 */
        float v = (float)mant * 5.9604644775390625e-08f;
        memcpy(&u, &v, 4);
        u |= sign;
    }
    float v;
    memcpy(&v, &u, 4);
    return v;
}
float moe_ref_round_f16(float v) { return moe_ref_f16_bits_to_f32(moe_ref_f32_to_f16_bits(v)); }

/* tf32 (torch_dtype 1; the reference's cute::tfloat32_t, types.cuh:128-131): an Element held in 32
 * bits. Conversion from fp32 is cutlass::NumericConverter<tfloat32_t, float> of CUTLASS (a dependency
 * the reference fetches at its main branch, csrc/CMakeLists.txt:106-167, absent here; restated from its
 * published source): round to nearest, ties to even, at mantissa bit 13, infinities and NaNs
 * untouched. CUTLASS leaves the 13 lower bits undefined; they are cleared here. A tensor core reads
 * only the upper 19 bits of a tf32 operand: moe_ref_tf32_operand. */
float moe_ref_round_tf32(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7f800000u) != 0x7f800000u) u += 0x0fffu + ((u >> 13) & 1u);
    u &= 0xffffe000u;
    memcpy(&v, &u, 4);
    return v;
}
float moe_ref_tf32_operand(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    u &= 0xffffe000u;
    memcpy(&v, &u, 4);
    return v;
}

static inline float to_elem(float v, uint32_t dtype) {
    return dtype == 2 ? moe_ref_round_bf16(v) : dtype == 3 ? moe_ref_round_f16(v) : dtype == 1 ? moe_ref_round_tf32(v) : v;
}

/* Packed-buffer element i as fp32. */
static inline float load_elem(const void* p, size_t i, uint32_t dtype) {
    return dtype == 2 ? moe_ref_bf16_bits_to_f32(((const uint16_t*)p)[i])
         : dtype == 3 ? moe_ref_f16_bits_to_f32(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
static inline void store_elem(void* p, size_t i, float v, uint32_t dtype) {
    if (dtype == 2) ((uint16_t*)p)[i] = moe_ref_f32_to_bf16_bits(v);
    else if (dtype == 3) ((uint16_t*)p)[i] = moe_ref_f32_to_f16_bits(v);
    else if (dtype == 1) ((float*)p)[i] = moe_ref_round_tf32(v);
    else ((float*)p)[i] = v;
}
static void load_elems(const void* p, size_t off, size_t n, uint32_t dtype, float* dst) {
    if (dtype == 2) {
        const uint16_t* s = (const uint16_t*)p + off;
        for (size_t i = 0; i < n; ++i) dst[i] = moe_ref_bf16_bits_to_f32(s[i]);
    } else if (dtype == 3) {
        const uint16_t* s = (const uint16_t*)p + off;
        for (size_t i = 0; i < n; ++i) dst[i] = moe_ref_f16_bits_to_f32(s[i]);
    } else if (dtype == 1) {
        /* rows that feed a matrix product: what a tf32 tensor core reads of them */
        const float* s = (const float*)p + off;
        for (size_t i = 0; i < n; ++i) dst[i] = moe_ref_tf32_operand(s[i]);
    } else {
        memcpy(dst, (const float*)p + off, n * sizeof(float));
    }
}

void moe_ref_gate_loss(uint32_t S, uint32_t E, const float* probs, const uint32_t* expert_count,
                       float* mean_prob, float* mean_count, float* loss) {
    /* gate.cuh:608-635 adds each tile's column sums of the probabilities, divided by S, into gML;
     * :700-705 adds each tile's routed counts divided by S into gMeC; :763-773 sums
     * gML[e] * gMeC[e] / E. The reference's float atomics fix no summation order: sums here are
     * taken in double and compared within tolerance. */
    double total = 0.0;
    for (uint32_t e = 0; e < E; ++e) {
        double col = 0.0;
        for (uint32_t t = 0; t < S; ++t) col += (double)probs[(size_t)t * E + e];
        const double mp = col / (double)S;
        const double mc = (double)expert_count[e] / (double)S;
        if (mean_prob) mean_prob[e] = (float)mp;
        if (mean_count) mean_count[e] = (float)mc;
        total += mp * mc;
    }
    *loss = (float)(total / (double)E);
}

int moe_ref_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ derived sizes */
int moe_ref_derive(moe_ref_cfg* c) {
    if (!c || !c->S || !c->H || !c->I || !c->E || !c->k || c->k > c->E) return -1;
    if (c->S % 128 || c->H % 64 || c->I % 64 || !(c->capacity_factor >= 1.0)) return -1;
    if (c->dtype > 3) return -1;
    c->PX = (c->E + 63u) / 64u * 64u;                                   /* types.cuh:481 */
    double base = c->drop_tokens ? (double)((c->S + c->E - 1u) / c->E) : (double)c->S;
    c->EC = (uint32_t)ceil(base * c->capacity_factor * (double)c->k - 1e-9); /* types.cuh:498-499 */
    c->pEC = (c->EC + 127u) / 128u * 128u;                              /* types.cuh:500 */
    c->cap_rows = c->pEC < c->S ? c->pEC : c->S;
    return 0;
}

/* ------------------------------------------------------------------ C = A * B^T, fp32
 * A [M,K] (lda), B [N,K] (ldb), C [M,N] (ldc). Summation order is fixed and independent of the
 * thread count: eight interleaved partial sums over k (lane j takes k = j mod 8), then the eight
 * lanes are added in ascending order. Requires K % 8 == 0 (H and I are multiples of 64). */
typedef float v8f __attribute__((vector_size(32), aligned(4)));

static inline float hsum8(v8f v) {
    float s = v[0];
    for (int j = 1; j < 8; ++j) s += v[j];
    return s;
}

/* B is taken from a packed Element buffer (bf16 bits or fp32) starting at element b_off; two of
 * its rows at a time are widened to fp32 into brow (2*K floats, caller-provided) and swept over
 * every row of A, so B streams once per call. */
static void gemm_nt(size_t M, size_t N, size_t K, const float* A, size_t lda, const void* Bp,
                    size_t b_off, uint32_t b_dtype, size_t ldb, float* C, size_t ldc, float* brow) {
    float* b0 = brow;
    float* b1 = brow + K;
    for (size_t n = 0; n < N; n += 2) {
        const int two = n + 1 < N;
        load_elems(Bp, b_off + n * ldb, K, b_dtype, b0);
        if (two) load_elems(Bp, b_off + (n + 1) * ldb, K, b_dtype, b1);
        else memset(b1, 0, K * sizeof(float));
        size_t m = 0;
        for (; m + 4 <= M; m += 4) {
            const float* a0 = A + (m + 0) * lda;
            const float* a1 = A + (m + 1) * lda;
            const float* a2 = A + (m + 2) * lda;
            const float* a3 = A + (m + 3) * lda;
            v8f c00 = {0}, c01 = {0}, c10 = {0}, c11 = {0}, c20 = {0}, c21 = {0}, c30 = {0}, c31 = {0};
            for (size_t kk = 0; kk < K; kk += 8) {
                v8f vb0 = *(const v8f*)(b0 + kk), vb1 = *(const v8f*)(b1 + kk);
                v8f va0 = *(const v8f*)(a0 + kk), va1 = *(const v8f*)(a1 + kk);
                v8f va2 = *(const v8f*)(a2 + kk), va3 = *(const v8f*)(a3 + kk);
                c00 += va0 * vb0; c01 += va0 * vb1;
                c10 += va1 * vb0; c11 += va1 * vb1;
                c20 += va2 * vb0; c21 += va2 * vb1;
                c30 += va3 * vb0; c31 += va3 * vb1;
            }
            C[(m + 0) * ldc + n] = hsum8(c00); C[(m + 1) * ldc + n] = hsum8(c10);
            C[(m + 2) * ldc + n] = hsum8(c20); C[(m + 3) * ldc + n] = hsum8(c30);
            if (two) {
                C[(m + 0) * ldc + n + 1] = hsum8(c01); C[(m + 1) * ldc + n + 1] = hsum8(c11);
                C[(m + 2) * ldc + n + 1] = hsum8(c21); C[(m + 3) * ldc + n + 1] = hsum8(c31);
            }
        }
        for (; m < M; ++m) {
            const float* a0 = A + m * lda;
            v8f c0 = {0}, c1 = {0};
            for (size_t kk = 0; kk < K; kk += 8) {
                v8f va = *(const v8f*)(a0 + kk);
                c0 += va * *(const v8f*)(b0 + kk);
                c1 += va * *(const v8f*)(b1 + kk);
            }
            C[m * ldc + n] = hsum8(c0);
            if (two) C[m * ldc + n + 1] = hsum8(c1);
        }
    }
}

/* ------------------------------------------------------------------ gate */
void moe_ref_gate_logits(uint32_t S, uint32_t H, uint32_t E, const float* x, const float* wg,
                         float* logits) {
    /* gate.cuh:526-534: one GEMM, fp32 accumulator. */
#pragma omp parallel
    {
        float* brow = (float*)malloc(2 * (size_t)H * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t t0 = 0; t0 < (int64_t)S; t0 += 64) {
            size_t rows = (size_t)S - (size_t)t0 < 64 ? (size_t)S - (size_t)t0 : 64;
            if (brow) gemm_nt(rows, E, H, x + (size_t)t0 * H, H, wg, 0, 0, H, logits + (size_t)t0 * E, E, brow);
        }
        free(brow);
    }
}

void moe_ref_softmax(uint32_t S, uint32_t E, const float* logits, float* probs) {
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < (int64_t)S; ++t) {
        const float* l = logits + (size_t)t * E;
        float* p = probs + (size_t)t * E;
        /* gate.cuh:574-580: online running max m and denominator d over the E real experts. */
        float d = 0.0f, m = -INFINITY;
        for (uint32_t e = 0; e < E; ++e) {
            const float pm = m;
            m = fmaxf(m, l[e]);
            d = fmaf(d, expf(pm - m), expf(l[e] - m));
        }
        /* gate.cuh:581-584 */
        for (uint32_t e = 0; e < E; ++e) p[e] = expf(l[e] - m) / d;
    }
}

void moe_ref_topk(uint32_t S, uint32_t E, uint32_t k, const float* logits, const float* probs,
                  int32_t* topk_expert, float* topk_prob, float* combine_den) {
#pragma omp parallel
    {
        uint8_t* taken = (uint8_t*)malloc(E);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < (int64_t)S; ++t) {
            const float* l = logits + (size_t)t * E;
            const float* p = probs + (size_t)t * E;
            memset(taken, 0, E);
            float den = 0.0f;
            /* gate.cuh:654-670: k rounds; strict '>' while scanning e upward keeps the lowest
             * index among equals. */
            for (uint32_t r = 0; r < k; ++r) {
                float best = -INFINITY;
                uint32_t arg = 0;
                int found = 0;
                for (uint32_t e = 0; e < E; ++e) {
                    /* the first untaken expert seeds the round so that a row holding -inf or NaN
                     * logits still selects k distinct experts */
                    if (!taken[e] && (!found || l[e] > best)) { best = l[e]; arg = e; found = 1; }
                }
                taken[arg] = 1;
                topk_expert[(size_t)t * k + r] = (int32_t)arg;
                topk_prob[(size_t)t * k + r] = p[arg];
                den += p[arg];
            }
            combine_den[t] = den;
        }
        free(taken);
    }
}

void moe_ref_slots(uint32_t S, uint32_t E, uint32_t k, uint32_t EC, uint32_t cap_rows,
                   const int32_t* topk_expert, int32_t* topk_slot, uint32_t* expert_count,
                   int32_t* slot_token) {
    memset(expert_count, 0, (size_t)E * sizeof(uint32_t));
    for (size_t i = 0; i < (size_t)E * cap_rows; ++i) slot_token[i] = -1;
    /* gate.cuh:678-718 with tiles taken in index order: rank among the tokens routed to the same
     * expert, in token order; keep iff rank < EC (gate.cuh:715). */
    for (uint32_t t = 0; t < S; ++t) {
        for (uint32_t r = 0; r < k; ++r) {
            const uint32_t e = (uint32_t)topk_expert[(size_t)t * k + r];
            const uint32_t rank = expert_count[e]++;
            if (rank < EC && rank < cap_rows) {
                topk_slot[(size_t)t * k + r] = (int32_t)rank;
                slot_token[(size_t)e * cap_rows + rank] = (int32_t)t;
            } else {
                topk_slot[(size_t)t * k + r] = -1;
            }
        }
    }
}

/* ------------------------------------------------------------------ activation */
static inline float act_fn(float v, uint32_t act) {
    if (act == 0) return v > 0.0f ? v : 0.0f;                       /* cutlass ReLU<float>  */
    return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));   /* cutlass GELU<float>: erf form */
}

/* ------------------------------------------------------------------ whole layer */
int moe_ref_forward(const moe_ref_cfg* c, const void* iP, void* oP, moe_ref_views* views,
                    int logits_given, const uint8_t* token_mask) {
    if (!c || !iP || !oP) return -1;
    const size_t S = c->S, H = c->H, I = c->I, E = c->E, k = c->k, PX = c->PX, CR = c->cap_rows;
    const uint32_t dt = c->dtype;
    if (logits_given && (!views || !views->logits)) return -1;

    const size_t off_wg = S * H, off_up = off_wg + PX * H, off_dn = off_up + E * I * H;
    const size_t off_bu = off_dn + E * H * I, off_bd = off_bu + E * I;
    const size_t off_out = S * PX;

    float* x = (float*)malloc(S * H * sizeof(float));
    float* logits = (float*)malloc(S * E * sizeof(float));
    float* probs = (float*)malloc(S * E * sizeof(float));
    int32_t* tk_e = (int32_t*)malloc(S * k * sizeof(int32_t));
    float* tk_p = (float*)malloc(S * k * sizeof(float));
    float* den = (float*)malloc(S * sizeof(float));
    int32_t* tk_s = (int32_t*)malloc(S * k * sizeof(int32_t));
    uint32_t* cnt = (uint32_t*)malloc(E * sizeof(uint32_t));
    int32_t* s_tok = (int32_t*)malloc(E * CR * sizeof(int32_t));
    /* y rows of every kept (token, rank) pair, Element values held as fp32 */
    float* y_pair = (float*)calloc(S * k * H, sizeof(float));
    int rc = -1;
    if (!x || !logits || !probs || !tk_e || !tk_p || !den || !tk_s || !cnt || !s_tok || !y_pair) goto done;

    load_elems(iP, 0, S * H, dt, x);
    if (logits_given) {
        memcpy(logits, views->logits, S * E * sizeof(float));
    } else {
        float* wg = (float*)malloc(E * H * sizeof(float));
        if (!wg) goto done;
        load_elems(iP, off_wg, E * H, dt, wg); /* only the E real rows of Wg[PX,H] */
        moe_ref_gate_logits(c->S, c->H, c->E, x, wg, logits);
        free(wg);
    }
    moe_ref_softmax(c->S, c->E, logits, probs);
    /* gateOut[t, 0:E] = Element(p); padded columns hold the zero logits of zero weight rows
     * untouched by the softmax (gate.cuh:550,576-605) */
    for (size_t t = 0; t < S; ++t) {
        for (size_t e = 0; e < PX; ++e)
            store_elem(oP, t * PX + e, e < E ? probs[t * E + e] : 0.0f, dt);
    }
    moe_ref_topk(c->S, c->E, c->k, logits, probs, tk_e, tk_p, den);
    moe_ref_slots(c->S, c->E, c->k, c->EC, c->cap_rows, tk_e, tk_s, cnt, s_tok);

    /* ---- experts: os/processor/processor.cuh:706-741 ---- */
    {
        /* work list: (expert, first row) blocks of RB kept rows */
        const size_t RB = 64;
        size_t n_tasks = 0;
        for (size_t e = 0; e < E; ++e) {
            size_t kept = cnt[e] < c->EC ? cnt[e] : c->EC; /* packet.cuh:85,112-113 */
            if (kept > CR) kept = CR;
            n_tasks += (kept + RB - 1) / RB;
        }
        uint32_t* task_e = (uint32_t*)malloc((n_tasks + 1) * sizeof(uint32_t));
        uint32_t* task_r = (uint32_t*)malloc((n_tasks + 1) * sizeof(uint32_t));
        if (!task_e || !task_r) { free(task_e); free(task_r); goto done; }
        n_tasks = 0;
        for (size_t e = 0; e < E; ++e) {
            size_t kept = cnt[e] < c->EC ? cnt[e] : c->EC;
            if (kept > CR) kept = CR;
            for (size_t r0 = 0; r0 < kept; r0 += RB) { task_e[n_tasks] = (uint32_t)e; task_r[n_tasks++] = (uint32_t)r0; }
        }
        int alloc_fail = 0;
#pragma omp parallel
        {
            const size_t Kmax = H > I ? H : I;
            float* brow = (float*)malloc(2 * Kmax * sizeof(float));
            float* xa = (float*)malloc(RB * H * sizeof(float));
            float* h1 = (float*)malloc(RB * I * sizeof(float));
            float* yy = (float*)malloc(RB * H * sizeof(float));
            int32_t* rows_tok = (int32_t*)malloc(RB * sizeof(int32_t));
            if (!brow || !xa || !h1 || !yy || !rows_tok) {
#pragma omp atomic write
                alloc_fail = 1;
            } else {
#pragma omp for schedule(dynamic, 1)
                for (int64_t ti = 0; ti < (int64_t)n_tasks; ++ti) {
                    const size_t e = task_e[ti], r0 = task_r[ti];
                    size_t kept = cnt[e] < c->EC ? cnt[e] : c->EC;
                    if (kept > CR) kept = CR;
                    /* gather the rows of this block whose token the mask selects (packet.cuh:151-160) */
                    size_t nr = 0;
                    for (size_t r = r0; r < kept && r < r0 + RB; ++r) {
                        const int32_t tok = s_tok[e * CR + r];
                        if (token_mask && !token_mask[tok]) continue;
                        rows_tok[nr] = tok;
                        memcpy(xa + nr * H, x + (size_t)tok * H, H * sizeof(float));
                        ++nr;
                    }
                    if (!nr) continue;
                    /* h1 = Element(act(acc + bias))  (gemm.cuh:22-31, processor.cuh:475) */
                    gemm_nt(nr, I, H, xa, H, iP, off_up + e * I * H, dt, H, h1, I, brow);
                    for (size_t r = 0; r < nr; ++r)
                        for (size_t j = 0; j < I; ++j)
                            h1[r * I + j] = to_elem(act_fn(h1[r * I + j] + load_elem(iP, off_bu + e * I + j, dt),
                                                           c->hidden_act), dt);
                    /* y = Element(acc + bias), identity activation (types.cuh:461) */
                    gemm_nt(nr, H, I, h1, I, iP, off_dn + e * H * I, dt, I, yy, H, brow);
                    for (size_t r = 0; r < nr; ++r) {
                        const size_t tok = (size_t)rows_tok[r];
                        size_t rank = 0;
                        while (rank < k && tk_e[tok * k + rank] != (int32_t)e) ++rank;
                        float* dst = y_pair + (tok * k + rank) * H;
                        for (size_t j = 0; j < H; ++j)
                            dst[j] = to_elem(yy[r * H + j] + load_elem(iP, off_bd + e * H + j, dt), dt);
                    }
                }
            }
            free(brow); free(xa); free(h1); free(yy); free(rows_tok);
        }
        free(task_e); free(task_r);
        if (alloc_fail) goto done;
    }

    /* ---- combine: os/processor/processor.cuh:110-168 (k > 1), :170-203 (k == 1) ---- */
#pragma omp parallel for schedule(static)
    for (int64_t tt = 0; tt < (int64_t)S; ++tt) {
        const size_t t = (size_t)tt;
        /* moe.cuh:43-48: the output starts from zero */
        for (size_t j = 0; j < H; ++j) store_elem(oP, off_out + t * H + j, 0.0f, dt);
        if (token_mask && !token_mask[t]) continue;
        if (k == 1) {
            if (tk_s[t] >= 0)
                for (size_t j = 0; j < H; ++j) store_elem(oP, off_out + t * H + j, y_pair[t * H + j], dt);
            continue;
        }
        /* ascending expert index: one legal order of the reference's atomics */
        for (size_t e = 0; e < E; ++e) {
            size_t rank = 0;
            while (rank < k && tk_e[t * k + rank] != (int32_t)e) ++rank;
            if (rank == k || tk_s[t * k + rank] < 0) continue;
            const float scale = load_elem(oP, t * PX + e, dt);          /* Element(gateOut[t,e]) (:117) */
            const float* yrow = y_pair + (t * k + rank) * H;
            for (size_t j = 0; j < H; ++j) {
                const float v = to_elem(yrow[j] / den[t], dt);            /* (:135) */
                const float prod = to_elem(scale * v, dt);                /* (:146) */
                const float acc = load_elem(oP, off_out + t * H + j, dt);
                store_elem(oP, off_out + t * H + j, to_elem(acc + prod, dt), dt); /* (:157,165) */
            }
        }
    }

    if (views) {
        if (views->logits && !logits_given) memcpy(views->logits, logits, S * E * sizeof(float));
        if (views->probs) memcpy(views->probs, probs, S * E * sizeof(float));
        if (views->topk_expert) memcpy(views->topk_expert, tk_e, S * k * sizeof(int32_t));
        if (views->topk_prob) memcpy(views->topk_prob, tk_p, S * k * sizeof(float));
        if (views->combine_den) memcpy(views->combine_den, den, S * sizeof(float));
        if (views->topk_slot) memcpy(views->topk_slot, tk_s, S * k * sizeof(int32_t));
        if (views->expert_count) memcpy(views->expert_count, cnt, E * sizeof(uint32_t));
        if (views->slot_token) memcpy(views->slot_token, s_tok, E * CR * sizeof(int32_t));
    }
    rc = 0;
done:
    free(x); free(logits); free(probs); free(tk_e); free(tk_p); free(den); free(tk_s);
    free(cnt); free(s_tok); free(y_pair);
    return rc;
}
