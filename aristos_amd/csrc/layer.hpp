// Device-visible description of one MoE layer invocation: configuration, the caller's packed
// buffers sliced into their parts, and the library-owned arenas. Passed by value to every kernel.
#pragma once
#include <cstdint>

namespace kleos_amd {

constexpr int kGateTileTokens = 16;   // tokens per gate tile (one MFMA column block)
constexpr int kSuperTiles = 32;       // gate tiles per coarse count row (512 tokens)
constexpr int kMaxGateGroups = 16;    // 16 experts per group: up to 256 experts keep their logits in registers

struct LayerParams {
    // ---- configuration (derived as the reference's struct ACC, types.cuh:471-507)
    uint32_t S, H, I, E, k, PX, EC, cap_rows, act;
    uint32_t is_training;     // 1: the gate also produces its load-balancing loss
    uint32_t n_gate_tiles;    // S / 16
    uint32_t n_super;         // ceil(n_gate_tiles / 32)
    // ---- caller buffers, sliced as moe.cuh:92-98
    const void* x;            // [S, H]
    const void* wg;           // [PX, H]
    const void* w_up;         // [E][I, H]
    const void* w_down;       // [E][H, I]
    const void* b_up;         // [E][I]
    const void* b_down;       // [E][H]
    void* gate_out;           // [S, PX]
    void* moe_out;            // [S, H]
    // ---- routing arenas (reference: Bookkeeping tP/eC, types.cuh:836-842)
    float* logits;            // [S, E]
    int32_t* topk_expert;     // [S, k]
    float* topk_prob;         // [S, k]
    float* combine_den;       // [S]
    int32_t* topk_slot;       // [S, k]  in-tile rank after the gate, final slot or -1 after slotting
    uint32_t* tile_count;     // [n_gate_tiles, E]   tokens of each 16-token tile routed to e
    uint32_t* super_count;    // [2][n_super, E]     the same summed over 32 tiles; two epochs
    uint32_t* expert_count;   // [E]
    int32_t* slot_token;      // [E, cap_rows]
    // ---- gate logits as a tiled product (16-bit Elements, more than 64 experts)
    float* gate_partial;      // [gate_splits][S, PX] fp32 sums over ranges of the hidden dimension
    uint32_t gate_splits;     // 0: the gate computes its logits per 16-token tile, without this array
    // ---- training-mode gate loss (reference: gML / gMeC / gL, types.cuh:940-958)
    float* tile_prob;         // [n_gate_tiles, E]  sum of the tile's 16 probabilities of expert e
    float* super_prob;        // [n_super, E]       the same summed over 32 tiles
    float* gate_loss;         // [E] mean probability | [E] mean routed count | [1] loss
    // ---- intermediate activations (reference: xM buffer, types.cuh:976-982)
    void* h1;                 // [E][cap_rows, I]
    void* y;                  // 4-byte Elements: [E][cap_rows, H]; 16-bit Elements: [E][ceil(H / 256)][cap_rows, 256] (y_offset)
    // ---- scheduler state of the persistent kernel
    uint32_t* sched;          // counters, see the scheduler section of kernels.hip
    unsigned long long* stamps;   // [workgroups][8] 100 MHz wall-clock stamps of the phase boundaries
    uint32_t epoch;           // launch parity, selects the live half of double-buffered counters
    unsigned long long wait_ticks;   // bound of every in-kernel wait, in ticks of the 100 MHz wall clock
};

// Where the down-projection's result for row `slot` of expert `e`, column `col`, sits in `y`, in Elements.
// 16-bit Elements keep y in pieces of kOutPiece columns - the width of an output tile - so that a tile's
// rows are one contiguous run of memory: the down-projection of a layer of many small experts writes
// several hundred MB in 128-row tiles, and written as 512-byte pieces 14 KB apart these stores cost the
// phase a twentieth more than written in one piece (256-expert top-8 shape: 2 825 against 2 870 us per
// forward). The combine reads a row as ceil(H / kOutPiece) pieces instead of one run, at the same speed.
constexpr uint32_t kOutPiece = 256;
__host__ __device__ inline size_t y_expert_elems(uint32_t cap_rows, uint32_t H, uint32_t elem_bytes) {
    const uint32_t Hp = elem_bytes == 2 ? (H + kOutPiece - 1) / kOutPiece * kOutPiece : H;
    return size_t(cap_rows) * Hp;
}
__host__ __device__ inline size_t y_offset(uint32_t e, uint32_t slot, uint32_t col, uint32_t cap_rows, uint32_t H, uint32_t elem_bytes) {
    const size_t base = size_t(e) * y_expert_elems(cap_rows, H, elem_bytes);
    if (elem_bytes != 2) return base + size_t(slot) * H + col;
    return base + size_t(col / kOutPiece) * cap_rows * kOutPiece + size_t(slot) * kOutPiece + col % kOutPiece;
}

}  // namespace kleos_amd
