/*
 * moe_ref.h — TEST INFRASTRUCTURE. CPU restatement of the Kleos/FlashDMoE single-GPU MoE-layer
 * forward (gate -> top-k -> capacity-bounded slots -> expert FFN -> weighted combine).
 *
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may link or call this; the
 * product library never does. See moe_ref.c for the reference file:line each function follows and
 * for what pins it.
 */
#ifndef MOE_REF_H
#define MOE_REF_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct moe_ref_cfg {
    uint32_t S, H, I, E, k;
    double capacity_factor;
    uint32_t drop_tokens;   /* 0 | 1 */
    uint32_t hidden_act;    /* 0 relu | 1 erf-gelu */
    uint32_t dtype;         /* 0 fp32 | 2 bf16 | 3 fp16 (Element) */
    /* derived by moe_ref_derive */
    uint32_t PX, EC, pEC, cap_rows;
} moe_ref_cfg;

/* Fills PX, EC, pEC, cap_rows. Returns 0, or -1 on an invalid shape. */
int moe_ref_derive(moe_ref_cfg* c);

/* Element helpers: round-to-nearest-even fp32 -> bf16 -> fp32, and raw conversions. */
float moe_ref_round_bf16(float v);
uint16_t moe_ref_f32_to_bf16_bits(float v);
float moe_ref_bf16_bits_to_f32(uint16_t b);
float moe_ref_round_f16(float v);
uint16_t moe_ref_f32_to_f16_bits(float v);
float moe_ref_f16_bits_to_f32(uint16_t b);
/* tf32 held in 32 bits: fp32 rounded to 10 mantissa bits (ties to even, lower 13 bits cleared), and
 * what a tensor core reads of a 32-bit operand (lower 13 bits cleared, no rounding). */
float moe_ref_round_tf32(float v);
float moe_ref_tf32_operand(float v);

/* logits[t,e] = sum_h x[t,h] * wg[e,h], fp32 accumulation. x [S,H], wg [E,H], logits [S,E]. */
void moe_ref_gate_logits(uint32_t S, uint32_t H, uint32_t E, const float* x, const float* wg,
                         float* logits);
/* Row softmax over the E real experts (fp32). */
void moe_ref_softmax(uint32_t S, uint32_t E, const float* logits, float* probs);
/* k rounds of strict-greater arg-max over ascending expert index (ties -> lower index), on the fp32
 * logits. topk_expert [S,k] in selection order, topk_prob [S,k] = probs of the selected,
 * combine_den [S] = their fp32 sum accumulated in selection order. */
void moe_ref_topk(uint32_t S, uint32_t E, uint32_t k, const float* logits, const float* probs,
                  int32_t* topk_expert, float* topk_prob, float* combine_den);
/* Token-order slot assignment with capacity drop. topk_slot [S,k] (-1 = dropped),
 * expert_count [E] (all routed, dropped included), slot_token [E,cap_rows] (-1 where unused). */
void moe_ref_slots(uint32_t S, uint32_t E, uint32_t k, uint32_t EC, uint32_t cap_rows,
                   const int32_t* topk_expert, int32_t* topk_slot, uint32_t* expert_count,
                   int32_t* slot_token);

/* Training-mode load-balancing loss of the gate: mean_prob[e] = (sum_t probs[t,e]) / S,
 * mean_count[e] = expert_count[e] / S (all routed tokens, dropped included),
 * loss = sum_e mean_prob[e] * mean_count[e] / E. mean_prob, mean_count [E] may be NULL. */
void moe_ref_gate_loss(uint32_t S, uint32_t E, const float* probs, const uint32_t* expert_count,
                       float* mean_prob, float* mean_count, float* loss);

typedef struct moe_ref_views {
    float* logits;          /* [S,E]   out (or in when logits_given != 0) */
    float* probs;           /* [S,E]   out, fp32 softmax                  */
    int32_t* topk_expert;   /* [S,k]   out */
    float* topk_prob;       /* [S,k]   out */
    float* combine_den;     /* [S]     out */
    int32_t* topk_slot;     /* [S,k]   out */
    uint32_t* expert_count; /* [E]     out */
    int32_t* slot_token;    /* [E,cap_rows] out */
} moe_ref_views;

/*
 * Whole layer on the packed Element buffers (same layout the GPU library takes):
 *   iP: x[S,H] | Wg[PX,H] | Wup[E][I,H] | Wdown[E][H,I] | bup[E][I] | bdown[E][H]
 *   oP: gateOut[S,PX] | moeOut[S,H]
 * logits_given != 0: views->logits is taken as the fp32 gate logits instead of being computed, so
 * that routing and outputs can be checked "given the same fp32 logits".
 * token_mask (may be NULL): [S] bytes; when given, expert FFNs and the combine are evaluated only
 * for tokens with a non-zero byte (their moeOut rows are exact, all other rows are left zero);
 * gate and routing are always evaluated for every token.
 * Any pointer inside views may be NULL (the stage's result is then kept internal). views itself
 * may be NULL. Returns 0, or -1 on allocation failure / bad arguments.
 */
int moe_ref_forward(const moe_ref_cfg* c, const void* iP, void* oP, moe_ref_views* views,
                    int logits_given, const uint8_t* token_mask);

/* Number of OpenMP threads the oracle will use. */
int moe_ref_threads(void);

#ifdef __cplusplus
}
#endif
#endif
