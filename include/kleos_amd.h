/*
 * kleos_amd.h — C ABI of the MI355X-native fused MoE forward.
 *
 * This is the drop-in boundary for the single-GPU (expert-parallel degree 1) MoE layer forward of
 * Kleos/FlashDMoE. Every entry point names the reference interface it replaces. All pointers are
 * plain host or device pointers, sizes are in bytes or elements as stated; no C++ or framework
 * types cross this boundary. Every function returning int returns 0 on success and a non-zero
 * KLEOS_E* code on failure; the text of the last failure is available from kleos_last_error().
 *
 * Threading: like the reference (process-global isInitialized / hostBookkeeping / seqBit,
 * reference csrc/include/kleos/types.cuh:440,1011-1012) the library holds ONE context per process.
 * Calls are not re-entrant; forwards issued back-to-back on the library stream are ordered.
 */
#ifndef KLEOS_AMD_H
#define KLEOS_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes --------------------------------------------------------------------------- */
enum {
    KLEOS_OK = 0,
    KLEOS_EINVAL = 1,      /* bad argument / invalid configuration value          */
    KLEOS_ESTATE = 2,      /* "Not initialized!" / "Already Initialized"           */
    KLEOS_EUNSUPPORTED = 3,/* valid reference config this build does not implement */
    KLEOS_EHIP = 4,        /* a HIP runtime call failed                            */
    KLEOS_EIO = 5,         /* config file could not be read                        */
    KLEOS_EPARSE = 6       /* config JSON malformed or a required key is missing   */
};

/* ---- configuration -------------------------------------------------------------------------- */
/* torch_dtype enumeration of the reference (csrc/kleos_config.schema.json:64-68). tf32 (the value the
 * reference ships, csrc/kleos_config.json:15) is an Element stored in 32 bits whose matrix products
 * use 10 mantissa bits of each operand (csrc/include/kleos/types.cuh:128-131, cute::tfloat32_t). CDNA4
 * has no tf32 matrix instruction: the products run on the fp32 matrix instructions with the lower 13
 * mantissa bits of the operands cleared, which gives the products a tf32 tensor core gives, and every
 * Element the layer writes (gateOut, moeOut, the activations between the projections) is fp32 rounded
 * to 10 mantissa bits, ties to even, lower bits zero. Buffers are packed as for fp32. */
enum { KLEOS_DTYPE_FP32 = 0, KLEOS_DTYPE_TF32 = 1, KLEOS_DTYPE_BF16 = 2, KLEOS_DTYPE_FP16 = 3 };
/* hidden_act enumeration of the reference (csrc/kleos_config.schema.json:29-33). */
enum { KLEOS_ACT_RELU = 0, KLEOS_ACT_GELU = 1 };

/*
 * The keys of kleos_config.json (reference csrc/kleos_config.schema.json:5-72) followed by the
 * constants the reference derives from them at compile time in struct ACC
 * (csrc/include/kleos/types.cuh:471-507). The reference consumes the JSON at CMake configure time
 * (csrc/CMakeLists.txt:186-252); here it is read at run time.
 */
typedef struct kleos_config {
    /* -- JSON keys -- */
    double   capacity_factor;   /* reference: integer >= 1; this build also takes real values   */
    uint32_t drop_tokens;       /* 0 | 1                                                         */
    uint32_t expert_top_k;
    uint32_t global_batch;      /* parsed, unused: feeds only the reference's placement models   */
    uint32_t is_training;       /* 0 | 1                                                         */
    uint32_t hidden_act;        /* KLEOS_ACT_*                                                   */
    uint32_t hidden_size;       /* H                                                             */
    uint32_t intermediate_size; /* I  ("P" in the reference)                                     */
    uint32_t mini_batch;
    uint32_t moe_frequency;     /* parsed, unused                                                */
    uint32_t num_experts;       /* E                                                             */
    uint32_t num_layers;        /* parsed, unused                                                */
    uint32_t sequence_len;
    uint32_t torch_dtype;       /* KLEOS_DTYPE_*                                                 */
    uint32_t vocab_size;        /* parsed, unused                                                */
    /* -- derived (types.cuh:471-507) -- */
    uint32_t S;                 /* tokens = sequence_len * mini_batch              (:471)        */
    uint32_t H, I, E, k;
    uint32_t PX;                /* experts padded to a multiple of 64              (:481)        */
    uint32_t EC;                /* expert capacity                                 (:498-499)    */
    uint32_t pEC;               /* EC padded to a multiple of 128                  (:500)        */
    uint32_t cap_rows;          /* min(pEC, S): row stride of every per-expert buffer. An expert
                                 * never holds more than S tokens, so without token dropping
                                 * (EC = S*cf*k) the arenas are sized by S instead.              */
    uint32_t elem_bytes;        /* sizeof(Element): 4 (fp32) or 2 (bf16, fp16)                   */
    /* Element offsets into the packed input buffer iP (csrc/include/kleos/moe/moe.cuh:92-96,
     * csrc/main.cu:23-28) and the packed output buffer oP (moe.cuh:97-98). */
    uint64_t off_x, off_gate_w, off_w_up, off_w_down, off_b_up, off_b_down, in_elems;
    uint64_t off_gate_out, off_moe_out, out_elems;
} kleos_config_t;

/* Parse a kleos_config.json text / file into cfg (keys only, no derivation, no validation beyond
 * JSON well-formedness and presence of the schema's required keys). */
int kleos_config_parse_string(const char* json_text, kleos_config_t* cfg);
int kleos_config_parse_file(const char* path, kleos_config_t* cfg);
/* Fill cfg with the shipped defaults of the reference (csrc/kleos_config.json:1-17) except
 * torch_dtype = bf16. */
void kleos_config_defaults(kleos_config_t* cfg);
/* Validate the keys and fill the derived fields. Enforces the reference's static_asserts
 * (csrc/include/kleos/bootstrap.cuh:542-545; types.cuh:479,496-497): S % 128 == 0, I % 64 == 0,
 * H % 64 == 0, k <= E, E <= 65535, capacity_factor >= 1. */
int kleos_config_derive(kleos_config_t* cfg);

/* ---- lifecycle ------------------------------------------------------------------------------ */
/* Replaces kleos::initialize() (csrc/include/kleos/bootstrap.cuh:533-547): validates the config,
 * selects the device, creates the library stream and allocates every scratch arena (routing
 * tables, intermediate activations, scheduler counters) the forward needs, as the reference's
 * Bookkeeping arenas are (bootstrap.cuh:377-391). Fails with KLEOS_ESTATE "Already Initialized",
 * and with KLEOS_EUNSUPPORTED for what this build leaves out: more than 512 experts, top-k
 * above 32 together with more than 256 experts. */
int kleos_initialize(const char* config_json_path);
int kleos_initialize_cfg(const kleos_config_t* cfg);
/* Replaces kleos::finalize() (bootstrap.cuh:562-588): drains the stream, frees every arena. */
int kleos_finalize(void);
int kleos_is_initialized(void);
/* Replaces kleos::getRank() (bootstrap.cuh:556-559): always 0 (expert-parallel degree 1).
 * Returns -1 when not initialised. */
int kleos_get_rank(void);
/* Replaces kleos::setDevice() (bootstrap.cuh:550-553): makes the library's GPU current. */
int kleos_set_device(void);
/* Copy of the active configuration (derived fields filled). */
int kleos_get_config(kleos_config_t* cfg);

/* ---- forward -------------------------------------------------------------------------------- */
/*
 * Replaces kleos::moe::forwardHost(iP, oP) (csrc/include/kleos/moe/moe.cuh:186-205).
 * iP: device pointer, packed Elements  x[S,H] | Wg[PX,H] | Wup[E][I,H] | Wdown[E][H,I] | bup[E][I] | bdown[E][H]
 * oP: device pointer, packed Elements  gateOut[S,PX] | moeOut[S,H]
 * Asynchronous on the library stream (the reference launches on kleosStream, types.cuh:1013); the
 * output is valid after kleos_stream_synchronize(). No host-side reset is needed between calls.
 * E == 1 runs the dense FFN (moe.cuh:197-204) ON THE SAME PACKED LAYOUT as every other expert
 * count: iP still carries the gate-weight block Wg[64,H] between x and Wup, and oP still starts
 * with gateOut[S,64] (all ones in column 0), i.e. off_w_up = S*H + 64*H and off_moe_out = S*64,
 * in_elems = S*H + 64*H + 2*I*H + I + H, out_elems = S*64 + S*H (kleos_get_config reports them).
 * This is the layout the reference's driver packs for any E (csrc/main.cu:23-30). It is NOT the
 * layout the reference's fffn kernel reads, iP = A | B1 | B2 | D1 | D2 and oP = C with no gate
 * blocks (csrc/include/kleos/moe/fffn.cuh:43-49): the reference's driver and its fffn disagree with
 * each other. kleos_moe_forward follows the driver; a caller that packs the fffn way calls
 * kleos_moe_forward_dense instead.
 */
int kleos_moe_forward(const void* iP, void* oP);
/*
 * num_experts == 1 only: the same dense FFN on the packing of the reference's fffn kernel
 * (csrc/include/kleos/moe/fffn.cuh:43-49, launched by forwardHost at moe.cuh:201-204):
 * iP: x[S,H] | Wup[I,H] | Wdown[H,I] | bup[I] | bdown[H]   (A | B1 | B2 | D1 | D2; no gate weights)
 * oP: moeOut[S,H]                                          (C; no gate output)
 * D2 follows the I entries of D1 (the reference steps over H entries there, fffn.cuh:49, which is the
 * same place whenever I == H). The gate still runs, on zero gate weights and into a gate output that
 * the library owns; moeOut has the bits kleos_moe_forward gives for the same operands. Asynchronous on
 * the library stream. KLEOS_ESTATE when the context holds more than one expert.
 */
int kleos_moe_forward_dense(const void* iP, void* oP);
/*
 * Replaces kleos::moe::forwardHostBench<skip,trials>(iP, oP, ms) (moe.cuh:146-184): `skip` untimed
 * launches, then `trials` launches bracketed by events on the library stream; *ms_per_launch is the
 * mean. Synchronises the stream before returning.
 */
int kleos_moe_forward_bench(const void* iP, void* oP, uint32_t skip, uint32_t trials,
                            float* ms_per_launch);
/*
 * No counterpart in the reference. For callers that cannot allocate device memory around a forward:
 * code under HIP stream capture, tight serving loops, harnesses that forbid hipMalloc. The same
 * forward as kleos_moe_forward (persistent launch, KLEOS_SCHEDULE_AUTO), but every library-owned array
 * (routing tables, the activations between the projections, scheduler counters) lives in a fixed
 * array of KLEOS_STATIC_SCRATCH_BYTES bytes (the last 256 hold a record of expired waits) in device
 * memory that each GPU holds from the moment the
 * library is loaded until the process ends. Needs no kleos_initialize and leaves an initialised
 * context alone; calls no hipMalloc / hipFree or any other allocating routine.
 *   cfg:    the JSON keys of the layer (derived fields are recomputed); a configuration whose arrays
 *           do not fit the scratch is refused with KLEOS_EUNSUPPORTED (the message states both sizes)
 *   iP, oP: as for kleos_moe_forward, on the current device
 *   stream: a hipStream_t (NULL: the default stream); the call enqueues a fill kernel that clears the
 *           counters, then the persistent kernel, and returns. The output is valid once the
 *           stream has drained.
 * All calls on one GPU share that GPU's array: calls that overlap on a GPU (two streams, two
 * threads) race and give wrong results; calls on one stream are ordered and safe, whatever their
 * configurations. The same holds for a kleos_moe_forward in flight on the library stream (which
 * does not wait for other streams): two persistent grids cannot be resident together, so the call
 * must not overlap it either. The first call for a layer on a device makes the runtime queries of a
 * launch plan (function attributes, occupancy) and, on a device's very first call, looks the array's
 * address up: make it outside stream capture, or call kleos_static_scratch_prepare first. Later calls
 * for that layer make no runtime queries. An expired in-kernel wait (the device was busy with other
 * kernels, or calls overlapped) is not reported by this call, which does not synchronise: ask
 * kleos_static_scratch_status.
 */
#define KLEOS_STATIC_SCRATCH_BYTES (32u << 20)
int kleos_moe_forward_static_scratch(const kleos_config_t* cfg, const void* iP, void* oP, void* stream);
/* No counterpart in the reference. Everything kleos_moe_forward_static_scratch needs before its first
 * launch of the layer `cfg` on the current device: the address of the device's scratch array and the
 * launch plan of the layer (kept for the sixteen most recent layers per device). Enqueues nothing,
 * allocates nothing. For callers whose first forward is recorded under stream capture. */
int kleos_static_scratch_prepare(const kleos_config_t* cfg);
/* No counterpart in the reference. Drains `stream` (a hipStream_t; NULL: the default stream), then
 * reports whether a bounded wait of the persistent kernel expired in any static-scratch call on the
 * current device since the last status call: KLEOS_OK, or KLEOS_EHIP (the text says whether it was
 * the most recent call or an earlier one), after which the record is cleared. The outputs of a call
 * with an expired wait are invalid. Allocates nothing. */
int kleos_static_scratch_status(void* stream);
/* Blocks until everything queued on the library stream has finished
 * (cudaStreamSynchronize(kleosStream) in the reference's callers, csrc/main.cu:64-70). */
int kleos_stream_synchronize(void);
/* The library stream as an opaque hipStream_t, for callers that want to order their own work
 * against it. NULL when not initialised. */
void* kleos_stream(void);

/* Which implementation kleos_moe_forward runs. 0 = one persistent launch with the in-kernel tile
 * scheduler (default); 1 = the same device functions as a sequence of separate launches, one per
 * phase (used to time phases in isolation). */
enum { KLEOS_MODE_FUSED = 0, KLEOS_MODE_PHASED = 1 };
int kleos_set_mode(int mode);
int kleos_get_mode(void);

/* How the persistent launch hands out expert tiles. The reference's scheduler is dynamic only
 * (csrc/include/kleos/os/scheduler.cuh); here the dynamic schedule (per-XCD ticket queues, readiness
 * counters, work stealing) has a static sibling: each XCD's workgroups stride through their queue
 * (all its up-projection tiles, then all its down-projection tiles) by a rank they take at the
 * start; a down-projection tile still checks the readiness counter of its row block, which is
 * normally complete long before. It spends nothing per tile on tickets or on writing results back
 * from the L2 for readers on other XCDs, and loses when the queues hold unequal work. KLEOS_SCHEDULE_AUTO (default) decides inside the kernel, from the
 * routed counts of the launch: static when no XCD's queue takes its workgroups more rounds of tiles
 * than the whole tile list would take spread over all workgroups.
 * KLEOS_SCHEDULE_STATIC still falls back to the dynamic schedule when the hardware did not place
 * the same number of workgroups on every XCD. Outputs are identical under every schedule. */
enum { KLEOS_SCHEDULE_AUTO = 0, KLEOS_SCHEDULE_DYNAMIC = 1, KLEOS_SCHEDULE_STATIC = 2 };
int kleos_set_schedule(int schedule);
int kleos_get_schedule(void);
/* The persistent kernel holds grid-wide barriers, so all its workgroups (one per compute unit) must
 * be resident together. The library sizes the grid from the occupancy the runtime reports for an
 * otherwise idle device. What happens on a device that is busy with other kernels:
 *   plain launch (default): kleos_moe_forward returns KLEOS_OK; inside the kernel every barrier gives
 *     up after its time limit (3 s each unless kleos_debug_set_wait_ticks says otherwise), the grid
 *     drains, and the NEXT synchronising call - kleos_stream_synchronize, kleos_moe_forward_bench,
 *     kleos_gate_loss - returns KLEOS_EHIP with "a bounded wait on the tile scheduler expired"; the
 *     outputs of that forward are invalid and the scheduler state has been reset.
 *   kleos_set_cooperative_launch(1): the kernel goes through hipLaunchCooperativeKernel, the runtime
 *     itself checks at every launch that the grid fits, and kleos_moe_forward ITSELF returns KLEOS_EHIP
 *     (the text names hipErrorCooperativeLaunchTooLarge) without launching anything. Measured: about
 *     14 us more per launch, which is why it is off by default.
 *   kleos_moe_forward_static_scratch: plain launch; kleos_static_scratch_status reports the expiry.
 * The reference launches its persistent kernel plainly (moe.cuh:170, 198) and does not check. */
int kleos_set_cooperative_launch(int on);
/* The schedule the most recent persistent launch took: KLEOS_SCHEDULE_DYNAMIC or
 * KLEOS_SCHEDULE_STATIC. Synchronises the library stream. KLEOS_ESTATE before the first launch. */
int kleos_schedule_taken(int* schedule);

/* ---- inspection (no counterpart in the reference, which exposes only gateOut and moeOut) ---- */
/*
 * Device pointers to the routing state left by the most recent forward, for parity checks of the
 * routing against fp32 logits. The arrays live in library-owned arenas and are overwritten by the
 * next forward; copy them out after kleos_stream_synchronize().
 */
typedef struct kleos_debug_views {
    const float*    logits;       /* [S, E]  fp32 gate logits (before softmax)                        */
    const int32_t*  topk_expert;  /* [S, k]  selected experts in selection order (best first)        */
    const float*    topk_prob;    /* [S, k]  fp32 softmax probability of each selected expert        */
    const float*    combine_den;  /* [S]     sum of the k selected probabilities (reference "mCw")   */
    const int32_t*  topk_slot;    /* [S, k]  slot inside the expert's buffer, or -1 when dropped     */
    const uint32_t* expert_count; /* [E]     tokens routed to each expert, dropped ones included     */
    const int32_t*  slot_token;   /* [E, cap_rows] token held by each slot (valid for slot < min(count,EC)) */
} kleos_debug_views_t;
int kleos_moe_debug_views(kleos_debug_views_t* views);
/* Drains the library stream, then copies `bytes` from a device pointer (one of the views above, or
 * any device buffer) into host memory. A convenience for callers without a HIP runtime binding. */
int kleos_debug_copy_to_host(void* host_dst, const void* device_src, size_t bytes);

/* Per-phase device time of the most recent kleos_moe_forward_bench, in milliseconds per launch:
 * [0] gate, [1] slotting, [2] up-projection, [3] down-projection, [4] combine.
 * KLEOS_MODE_PHASED: event-timed kernels, averaged over the trials. KLEOS_MODE_FUSED: taken from
 * wall-clock stamps every workgroup of the last persistent launch leaves at its phase boundaries
 * (each phase through the grid barrier that ends it); the two projections interleave in one phase,
 * reported in [2] with [3] = 0. */
int kleos_phase_times(float ms[5]);
/* Tile-scheduler statistics of the last launch of the most recent kleos_moe_forward_bench in
 * KLEOS_MODE_FUSED (the persistent kernel keeps them per workgroup; the reference has no
 * counterpart): [0..2] mean milliseconds a workgroup spent fetching tasks, waiting for an
 * unfinished dependency, publishing finished tiles; [3] expert tiles executed; [4] tiles handed out
 * before their inputs were complete; [5] tiles taken from another XCD's queue. */
int kleos_scheduler_stats(double stats[6]);
/* Replaces kleos::mT (csrc/include/kleos/throughput.cuh:104-170), the probe the reference runs at
 * start-up to rate a device: one expert at full padded capacity (pEC rows) through the up-projection,
 * activation and down-projection of the configured sizes, `trials` times on the library stream after
 * two warm-up rounds. *median_ms receives the median latency of a round, *throughput its reciprocal
 * (experts per millisecond), the figure the reference stores in WorkerAttribute::throughput. Allocates
 * and frees its own operands; the context's state is untouched. */
int kleos_measure_throughput(uint32_t trials, float* median_ms, float* throughput);
/* The same probe, which also copies the first y_bytes of its result y[pEC, H] (Elements, row-major)
 * to host memory before it frees its operands. The probe fills x, both weight matrices and both
 * bias vectors with the byte 0x3c, so every Element has one value v (bf16 0.01147, fp16 1.0586,
 * fp32 0.011489) and every result element is Element(I * Element(act(H*v*v + v)) * v + v): what the
 * reference's probe computes is never looked at either (throughput.cuh:104-170 times the kernel of
 * moe/expert.cuh:203-372), this lets a test check the launch geometry of the probe. */
int kleos_measure_throughput_output(uint32_t trials, float* median_ms, float* throughput, void* y_host,
                                    size_t y_bytes);
/* Training mode (is_training: 1): the load-balancing loss of the gate of the most recent forward,
 * which the reference leaves in its bookkeeping arena (gML, gMeC, gL; csrc/include/kleos/types.cuh:
 * 940-958, computed at moe/gate.cuh:608-635, 700-705, 763-773): mean_prob[e] = mean over the tokens
 * of the softmax probability of expert e, mean_count[e] = tokens routed to e (dropped included) / S,
 * *loss = sum_e mean_prob[e] * mean_count[e] / E. mean_prob and mean_count ([E] floats) may be
 * NULL. Synchronises the library stream. KLEOS_ESTATE when the context is not in training mode. */
int kleos_gate_loss(float* loss, float* mean_prob, float* mean_count);
/* Raw phase stamps of the most recent persistent launch (KLEOS_MODE_FUSED), for timing studies; the
 * reference has no counterpart. Synchronises the library stream, then copies, for each of the first
 * min(*n_workgroups, max_workgroups) workgroups, 8 readings of the 100 MHz device wall clock:
 * [0] kernel entry, [1] gate tiles done, [2] past barrier 1, [3] slots done, [4] past barrier 2,
 * [5] expert tiles done, [6] past barrier 3, [7] combine done. *n_workgroups receives the size of
 * the launch. */
int kleos_phase_stamps(unsigned long long* stamps, uint32_t max_workgroups, uint32_t* n_workgroups);

/* ---- failure handling of the persistent launch (no counterpart in the reference, whose waits are
 * unbounded) ---- */
/* Every wait inside the persistent kernel (grid barriers, row-block readiness) gives up after this
 * many ticks of the device's 100 MHz wall clock (default 300 000 000 = 3 s; 0 restores the default):
 * the grid always drains, the synchronising call that follows returns KLEOS_EHIP, and the library
 * resets its scheduler counters so that the next forward behaves as on a fresh context. */
int kleos_debug_set_wait_ticks(unsigned long long ticks);
/* Makes the library count one persistent launch that never ran: the barrier counters then lag what
 * the next launch expects, every barrier of that launch runs into its time limit, and the launch
 * reports the expiry. For tests of the recovery path (with a small tick limit set first). */
int kleos_debug_skip_launch_number(void);

/* The tests' handle on kleos_static_scratch_status: later static-scratch calls run with this tick limit
 * on their in-kernel waits (0: the default) and as launch number `skip_launch_numbers` of their fresh
 * counters instead of 0, so that with a non-zero skip every barrier runs into the limit, every kernel
 * still exits, and the status call reports the expiry. (0, 0) restores normal operation. */
int kleos_debug_static_scratch_expiry(unsigned long long ticks, uint32_t skip_launch_numbers);
/* The code and message a failed HIP runtime call turns into at this boundary: KLEOS_OK for
 * hipSuccess (0), else KLEOS_EHIP with the runtime's name and description of `hip_error` in
 * kleos_last_error(). Touches no device: lets a test pin, for instance, what a refused cooperative
 * launch (hipErrorCooperativeLaunchTooLarge) looks like to a caller. */
int kleos_debug_map_hip_error(int hip_error);
/* Measurement probe with no counterpart in the reference and no part in the layer: one launch, on the
 * current device's null stream, of a loop of bf16 matrix instructions on operands held in registers
 * (eight wavefronts on every CU, no LDS or memory traffic inside the loop), timed by events. tile 32
 * issues 32x32x16 instructions, tile 16 issues 16x16x32; operands are random bf16 values of unit size,
 * or zeros. *ms: duration of the launch, *flop: its floating-point operations. What the matrix cores
 * sustain at the package's power cap, and how that depends on the instruction and on the data, is
 * what bounds the expert GEMM (bench.py --calib-mfma samples the socket power around it). Keeps
 * 16 MB of device memory until the process ends. */
int kleos_debug_mfma_probe(int tile, uint32_t iterations, int zero_operands, float* ms, double* flop);

/* ---- errors --------------------------------------------------------------------------------- */
/* Replaces the KLEOS_CHECK_CUDA / KLEOS_ASSERT message conventions (csrc/include/kleos/debug.cuh:
 * 19-43), which print and exit; the C ABI records the message and returns a code instead. */
const char* kleos_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* KLEOS_AMD_H */
