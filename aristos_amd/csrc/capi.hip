// The C ABI declared in include/kleos_amd.h: lifecycle, forward, bench, inspection.
//
// Mirrors the host side of the reference: kleos::initialize / finalize / getRank / setDevice
// (csrc/include/kleos/bootstrap.cuh:533-588) and kleos::moe::forwardHost / forwardHostBench
// (csrc/include/kleos/moe/moe.cuh:146-205), for one GPU and expert-parallel degree 1.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "common.hpp"
#include "kernels.hpp"

namespace kleos_amd {
namespace {

struct Context {
    kleos_config_t cfg{};
    int device = 0;
    int num_cus = 0;
    hipStream_t stream = nullptr;
    char* arena = nullptr;          // one allocation holding every library-owned buffer
    size_t arena_bytes = 0;
    LayerParams base{};             // configuration + arena pointers; caller buffers filled per call
    FusedPlan plan{};
    uint32_t launch_seq = 0;        // forwards issued, any mode (parity selects the live coarse counts)
    uint32_t fused_seq = 0;         // fused forwards issued (grid-barrier arrival base)
    int mode = KLEOS_MODE_FUSED;
    int schedule = KLEOS_SCHEDULE_AUTO;
    size_t zero_begin = 0, zero_end = 0;   // the part of the arena that holds counters (starts as zeros)
    char* dense_wg = nullptr;       // one expert: zero gate weights and a gate output owned by the library
    char* dense_gate_out = nullptr;
    float phase_ms[5] = {0, 0, 0, 0, 0};
    double sched_stats[6] = {0, 0, 0, 0, 0, 0};
};

Context* g_ctx = nullptr;   // one context per process, like the reference's global state

#define KLEOS_HIP(expr)                                                                         \
    do {                                                                                        \
        hipError_t e_ = (expr);                                                                 \
        if (e_ != hipSuccess)                                                                   \
            return fail(KLEOS_EHIP, "<%s:%d> %s:\n    %s: %s", __FILE__, __LINE__, #expr,       \
                        hipGetErrorName(e_), hipGetErrorString(e_));                            \
    } while (0)

constexpr uint32_t kMaxWorkgroups = 1024;   // persistent grid never exceeds CUs x 2
constexpr unsigned long long kDefaultWaitTicks = 300000000ull;   // 3 s of the 100 MHz wall clock

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct ArenaLayout {
    size_t logits, topk_expert, topk_prob, combine_den, topk_slot, tile_count, super_count,
        expert_count, slot_token, h1, y, sched, stamps, tile_prob, super_prob, gate_loss, gate_partial, dense_wg, dense_gate_out, total;
    size_t zero_begin, zero_end;   // range that must start as zeros
};

ArenaLayout layout_arena(const kleos_config_t& c, uint32_t n_tiles, uint32_t n_super, uint32_t gate_splits) {
    ArenaLayout L{};
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
    const size_t S = c.S, E = c.E, k = c.k, R = c.cap_rows;
    // counters first: they are the part cleared at initialisation
    // (the scheduler words come first: the error word then sits at the same place in every layout)
    L.zero_begin = off;
    L.sched = take(sched_words(c.E, c.cap_rows) * 4);
    L.super_count = take(2 * size_t(n_super) * E * 4);
    L.expert_count = take(E * 4);
    L.stamps = take(size_t(kMaxWorkgroups) * 16 * 8);
    L.gate_loss = take((2 * E + 1) * 4);
    L.zero_end = off;
    L.tile_prob = take(size_t(n_tiles) * E * 4);
    L.super_prob = take(size_t(n_super) * E * 4);
    L.logits = take(S * E * 4);
    L.topk_expert = take(S * k * 4);
    L.topk_prob = take(S * k * 4);
    L.combine_den = take(S * 4);
    L.topk_slot = take(S * k * 4);
    L.tile_count = take(size_t(n_tiles) * E * 4);
    L.slot_token = take(E * R * 4);
    L.h1 = take(E * R * size_t(c.I) * c.elem_bytes);
    L.y = take(E * y_expert_elems(uint32_t(R), c.H, c.elem_bytes) * c.elem_bytes);
    L.gate_partial = take(size_t(gate_splits) * S * c.PX * 4);
    // one expert: gate weights (zeros) and a gate output of the library's own, for callers that pack the
    // dense-FFN way, without either (kleos_moe_forward_dense)
    L.dense_wg = take(E == 1 ? size_t(c.PX) * c.H * c.elem_bytes : 0);
    L.dense_gate_out = take(E == 1 ? S * size_t(c.PX) * c.elem_bytes : 0);
    L.total = off;
    return L;
}

// After a synchronisation: did a persistent kernel give up waiting on its scheduler counters?
// A launch that gave up leaves the monotonic barrier counters, the member counts and the count of
// static launches short of what the launch numbers imply, so every counter goes back to zero and
// the launch numbers with them: the next forward starts from the state of a fresh context.
int check_scheduler(Context& c) {
    uint32_t flag = 0;
    hipError_t e = hipMemcpy(&flag, c.base.sched + sched_error_word(), 4, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail(KLEOS_EHIP, "scheduler check: %s", hipGetErrorString(e));
    if (flag) {
        e = hipMemset(c.arena + c.zero_begin, 0, c.zero_end - c.zero_begin);
        c.launch_seq = 0;
        c.fused_seq = 0;
        if (e != hipSuccess) return fail(KLEOS_EHIP, "scheduler reset: %s", hipGetErrorString(e));
        return fail(KLEOS_EHIP, "persistent kernel: a bounded wait on the tile scheduler expired; "
                                "the outputs of that launch are invalid (scheduler state reset)");
    }
    return KLEOS_OK;
}

int require_ctx(const char* who) {
    if (!g_ctx) return fail(KLEOS_ESTATE, "%s: Not initialized!", who);
    return KLEOS_OK;
}

// The caller's packed buffers, sliced as moe.cuh:92-98.
void bind_buffers(LayerParams& p, const kleos_config_t& cfg, const void* iP, void* oP) {
    const size_t eb = cfg.elem_bytes;
    const char* in = static_cast<const char*>(iP);
    char* out = static_cast<char*>(oP);
    p.x = in + cfg.off_x * eb;
    p.wg = in + cfg.off_gate_w * eb;
    p.w_up = in + cfg.off_w_up * eb;
    p.w_down = in + cfg.off_w_down * eb;
    p.b_up = in + cfg.off_b_up * eb;
    p.b_down = in + cfg.off_b_down * eb;
    p.gate_out = out + cfg.off_gate_out * eb;
    p.moe_out = out + cfg.off_moe_out * eb;
}

LayerParams bind(const Context& c, const void* iP, void* oP) {
    LayerParams p = c.base;
    bind_buffers(p, c.cfg, iP, oP);
    return p;
}

// The configuration part of the kernel parameters (a derived configuration).
void params_from_config(LayerParams& p, const kleos_config_t& cfg) {
    p.S = cfg.S; p.H = cfg.H; p.I = cfg.I; p.E = cfg.E; p.k = cfg.k; p.PX = cfg.PX;
    p.EC = cfg.EC; p.cap_rows = cfg.cap_rows; p.act = cfg.hidden_act;
    p.is_training = cfg.is_training;
    p.n_gate_tiles = cfg.S / kGateTileTokens;
    p.n_super = (p.n_gate_tiles + kSuperTiles - 1) / kSuperTiles;
    p.wait_ticks = kDefaultWaitTicks;
}

// The library-owned arrays of the kernel parameters, laid out in the memory at `a`.
void params_from_arena(LayerParams& p, char* a, const ArenaLayout& L) {
    p.logits = reinterpret_cast<float*>(a + L.logits);
    p.topk_expert = reinterpret_cast<int32_t*>(a + L.topk_expert);
    p.topk_prob = reinterpret_cast<float*>(a + L.topk_prob);
    p.combine_den = reinterpret_cast<float*>(a + L.combine_den);
    p.topk_slot = reinterpret_cast<int32_t*>(a + L.topk_slot);
    p.tile_count = reinterpret_cast<uint32_t*>(a + L.tile_count);
    p.super_count = reinterpret_cast<uint32_t*>(a + L.super_count);
    p.expert_count = reinterpret_cast<uint32_t*>(a + L.expert_count);
    p.slot_token = reinterpret_cast<int32_t*>(a + L.slot_token);
    p.tile_prob = reinterpret_cast<float*>(a + L.tile_prob);
    p.super_prob = reinterpret_cast<float*>(a + L.super_prob);
    p.gate_loss = reinterpret_cast<float*>(a + L.gate_loss);
    p.h1 = a + L.h1;
    p.y = a + L.y;
    p.sched = reinterpret_cast<uint32_t*>(a + L.sched);
    p.stamps = reinterpret_cast<unsigned long long*>(a + L.stamps);
    p.gate_partial = reinterpret_cast<float*>(a + L.gate_partial);
}

// Enqueues one forward. When ev is non-null (phased mode) it receives 6 recorded events that
// bracket the five phases.
int enqueue_forward(Context& c, const void* iP, void* oP, hipEvent_t* ev, bool dense_packing = false) {
    if (!iP || !oP) return fail(KLEOS_EINVAL, "forward: null buffer");
    if ((reinterpret_cast<uintptr_t>(iP) | reinterpret_cast<uintptr_t>(oP)) & 15u)
        return fail(KLEOS_EINVAL, "forward: iP and oP must be 16-byte aligned");
    LayerParams p = bind(c, iP, oP);
    if (dense_packing) {
        // iP = A | B1 | B2 | D1 | D2, oP = C (fffn.cuh:43-49): no gate weights, no gate output
        const kleos_config_t& g = c.cfg;
        const size_t eb = g.elem_bytes;
        const char* in = static_cast<const char*>(iP);
        p.x = in;
        p.w_up = in + size_t(g.S) * g.H * eb;
        p.w_down = static_cast<const char*>(p.w_up) + size_t(g.I) * g.H * eb;
        p.b_up = static_cast<const char*>(p.w_down) + size_t(g.H) * g.I * eb;
        p.b_down = static_cast<const char*>(p.b_up) + size_t(g.I) * eb;
        p.wg = c.dense_wg;
        p.gate_out = c.dense_gate_out;
        p.moe_out = oP;
    }
    p.epoch = c.launch_seq++;
    const int dt = int(c.cfg.torch_dtype);
    if (c.mode == KLEOS_MODE_FUSED) {
        KLEOS_HIP(launch_fused(p, c.plan, c.fused_seq++, c.schedule, c.stream));
        return KLEOS_OK;
    }
    if (ev) KLEOS_HIP(hipEventRecord(ev[0], c.stream));
    KLEOS_HIP(launch_gate(p, dt, c.num_cus, c.stream));
    if (ev) KLEOS_HIP(hipEventRecord(ev[1], c.stream));
    KLEOS_HIP(launch_slots(p, c.stream));
    if (ev) KLEOS_HIP(hipEventRecord(ev[2], c.stream));
    KLEOS_HIP(launch_expert_gemm(p, dt, 0, c.num_cus, c.stream));
    if (ev) KLEOS_HIP(hipEventRecord(ev[3], c.stream));
    KLEOS_HIP(launch_expert_gemm(p, dt, 1, c.num_cus, c.stream));
    if (ev) KLEOS_HIP(hipEventRecord(ev[4], c.stream));
    KLEOS_HIP(launch_combine(p, dt, c.stream));
    if (ev) KLEOS_HIP(hipEventRecord(ev[5], c.stream));
    return KLEOS_OK;
}

// ---------------------------------------------------------------- the entry point that allocates nothing
// Every library-owned array of a forward (routing tables, h1, y, scheduler counters, stamps) laid out
// in a fixed array in device memory instead of an arena from hipMalloc. Every GPU the library runs
// on holds its own copy of the array, at its own address, until the process ends. The last 256
// bytes of the array are not part of any layout: their first word is the sticky record of expired
// waits that kleos_static_scratch_status reads.
constexpr size_t kStaticScratchBytes = KLEOS_STATIC_SCRATCH_BYTES;
constexpr size_t kStaticScratchTail = 256;
constexpr size_t kStaticScratchUsable = kStaticScratchBytes - kStaticScratchTail;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// A plan of the persistent launch as a call found it, kept so that repeated calls with the same
// layer make no runtime queries.
struct CachedPlan {
    bool used = false;
    uint32_t dtype = 0, S = 0, H = 0, I = 0, E = 0, k = 0, EC = 0, cap_rows = 0, is_training = 0;
    FusedPlan plan{};
};
constexpr int kCachedPlans = 16;

// What a device needs once: the address of its copy of `scratch` (in host code the array's name is
// only a handle for hipGetSymbolAddress, never a device address) and its compute-unit count.
struct DeviceSetup {
    bool ready = false;
    char* scratch_ptr = nullptr;
    int num_cus = 0;
    bool gfx950 = false;
    CachedPlan plans[kCachedPlans];
    int next_plan = 0;
};
constexpr int kMaxDevices = 64;
DeviceSetup g_devices[kMaxDevices];
std::mutex g_devices_mutex;
// Test hooks of the static-scratch path (kleos_debug_static_scratch_expiry): a tick budget for its
// in-kernel waits and launch numbers to skip, which makes every barrier of its launches expire.
unsigned long long g_static_wait_ticks = 0;
uint32_t g_static_skip = 0;

// Looks the current device up (first call per device) or returns what was found then.
int device_setup(DeviceSetup** out) {
    int dev = -1;
    KLEOS_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(KLEOS_EUNSUPPORTED, "device ordinal %d is beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_devices_mutex);
    DeviceSetup& d = g_devices[dev];
    if (!d.ready) {
        void* ptr = nullptr;
        KLEOS_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(KLEOS_EHIP, "hipGetSymbolAddress returned a null address for the static scratch");
        hipDeviceProp_t prop;
        KLEOS_HIP(hipGetDeviceProperties(&prop, dev));
        d.scratch_ptr = static_cast<char*>(ptr);
        d.num_cus = prop.multiProcessorCount;
        d.gfx950 = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
        d.ready = true;
    }
    *out = &d;
    return KLEOS_OK;
}

// Clears the counter range of a layout. The thread that owns the error word first copies a set
// word into the sticky record, so that an expired wait of the previous call stays on record until
// kleos_static_scratch_status has reported it.
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* words, size_t n, size_t error_index, uint32_t* sticky) {
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += size_t(gridDim.x) * blockDim.x) {
        if (i == error_index && words[i] != 0u) *sticky = 1u;
        words[i] = 0u;
    }
}

// Everything a static-scratch call derives from its configuration before it touches the stream.
struct StaticCall {
    kleos_config_t cfg;
    DeviceSetup* dev = nullptr;
    LayerParams p{};
    ArenaLayout L{};
    FusedPlan plan{};
};

int prepare_static_call(const kleos_config_t* user_cfg, StaticCall& c) {
    c.cfg = *user_cfg;
    if (int rc = kleos_config_derive(&c.cfg)) return rc;
    if (const char* why = unsupported_reason(c.cfg.E, c.cfg.k)) return fail(KLEOS_EUNSUPPORTED, "%s", why);
    if (int rc = device_setup(&c.dev)) return rc;
    if (!c.dev->gfx950) return fail(KLEOS_EUNSUPPORTED, "the current device is not gfx950: this library is built for MI355X only");
    params_from_config(c.p, c.cfg);
    c.p.gate_splits = gate_splits_for(c.cfg.S, c.cfg.H, c.cfg.E, c.cfg.PX, int(c.cfg.torch_dtype), c.dev->num_cus);
    c.L = layout_arena(c.cfg, c.p.n_gate_tiles, c.p.n_super, c.p.gate_splits);
    if (c.L.total > kStaticScratchUsable)
        return fail(KLEOS_EUNSUPPORTED, "kleos_moe_forward_static_scratch: this configuration needs %zu bytes of library "
                    "memory, the static scratch holds %zu; use kleos_initialize + kleos_moe_forward", c.L.total,
                    kStaticScratchUsable);
    if (c.L.sched != 0) return fail(KLEOS_EHIP, "static scratch: the scheduler words must open the layout");
    params_from_arena(c.p, c.dev->scratch_ptr, c.L);
    // the plan of this layer: looked up, or made once (function attributes, occupancy query) and kept
    std::lock_guard<std::mutex> lock(g_devices_mutex);
    const kleos_config_t& g = c.cfg;
    for (CachedPlan& e : c.dev->plans)
        if (e.used && e.dtype == g.torch_dtype && e.S == g.S && e.H == g.H && e.I == g.I && e.E == g.E && e.k == g.k &&
            e.EC == g.EC && e.cap_rows == g.cap_rows && e.is_training == g.is_training) {
            c.plan = e.plan;
            return KLEOS_OK;
        }
    KLEOS_HIP(plan_fused(c.p, int(g.torch_dtype), c.dev->num_cus, &c.plan));
    if (c.plan.nwg > kMaxWorkgroups) return fail(KLEOS_EUNSUPPORTED, "persistent grid of %u workgroups exceeds %u", c.plan.nwg, kMaxWorkgroups);
    CachedPlan& e = c.dev->plans[c.dev->next_plan];
    c.dev->next_plan = (c.dev->next_plan + 1) % kCachedPlans;
    e.used = true; e.dtype = g.torch_dtype; e.S = g.S; e.H = g.H; e.I = g.I; e.E = g.E; e.k = g.k; e.EC = g.EC;
    e.cap_rows = g.cap_rows; e.is_training = g.is_training; e.plan = c.plan;
    return KLEOS_OK;
}

}  // namespace
}  // namespace kleos_amd

using namespace kleos_amd;

extern "C" int kleos_static_scratch_prepare(const kleos_config_t* user_cfg) {
    if (!user_cfg) return fail(KLEOS_EINVAL, "kleos_static_scratch_prepare: null config");
    StaticCall c;
    return prepare_static_call(user_cfg, c);
}

extern "C" int kleos_moe_forward_static_scratch(const kleos_config_t* user_cfg, const void* iP, void* oP, void* stream) {
    if (!user_cfg) return fail(KLEOS_EINVAL, "kleos_moe_forward_static_scratch: null config");
    if (!iP || !oP) return fail(KLEOS_EINVAL, "kleos_moe_forward_static_scratch: null buffer");
    if ((reinterpret_cast<uintptr_t>(iP) | reinterpret_cast<uintptr_t>(oP)) & 15u)
        return fail(KLEOS_EINVAL, "kleos_moe_forward_static_scratch: iP and oP must be 16-byte aligned");
    StaticCall c;
    if (int rc = prepare_static_call(user_cfg, c)) return rc;
    LayerParams& p = c.p;
    bind_buffers(p, c.cfg, iP, oP);
    // The array keeps what the last call left, of whatever configuration: every counter goes back
    // to zero (a fill kernel, which a stream capture records faithfully), and the launch runs as the
    // first one of a fresh arena.
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t words = (c.L.zero_end - c.L.zero_begin) / 4;
    uint32_t* sticky = reinterpret_cast<uint32_t*>(c.dev->scratch_ptr + kStaticScratchUsable);
    // (every layout starts with the scheduler words, so whatever call came before left its error word here)
    hipLaunchKernelGGL(zero_words_kernel, dim3(64), dim3(256), 0, s, reinterpret_cast<uint32_t*>(c.dev->scratch_ptr + c.L.zero_begin),
                       words, (c.L.sched - c.L.zero_begin) / 4 + size_t(sched_error_word()), sticky);
    KLEOS_HIP(hipGetLastError());
    p.epoch = 0;
    if (g_static_wait_ticks) p.wait_ticks = g_static_wait_ticks;
    KLEOS_HIP(launch_fused(p, c.plan, g_static_skip, KLEOS_SCHEDULE_AUTO, s));
    return KLEOS_OK;
}

extern "C" int kleos_static_scratch_status(void* stream) {
    DeviceSetup* dev = nullptr;
    if (int rc = device_setup(&dev)) return rc;
    KLEOS_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    // the word of the last launch (every layout keeps it at the same place), and the record of the launches before it
    const size_t error_offset = size_t(sched_error_word()) * 4;
    uint32_t now = 0, before = 0;
    KLEOS_HIP(hipMemcpy(&now, dev->scratch_ptr + error_offset, 4, hipMemcpyDeviceToHost));
    KLEOS_HIP(hipMemcpy(&before, dev->scratch_ptr + kStaticScratchUsable, 4, hipMemcpyDeviceToHost));
    if (!now && !before) return KLEOS_OK;
    const uint32_t zero = 0;
    KLEOS_HIP(hipMemcpy(dev->scratch_ptr + error_offset, &zero, 4, hipMemcpyHostToDevice));
    KLEOS_HIP(hipMemcpy(dev->scratch_ptr + kStaticScratchUsable, &zero, 4, hipMemcpyHostToDevice));
    return fail(KLEOS_EHIP, "kleos_moe_forward_static_scratch: a bounded wait of the persistent kernel expired in %s; "
                            "the outputs of that call are invalid (is the device busy with other kernels, or did calls overlap?)",
                now ? "the most recent call" : "an earlier call");
}

extern "C" int kleos_debug_static_scratch_expiry(unsigned long long ticks, uint32_t skip_launch_numbers) {
    g_static_wait_ticks = ticks;
    g_static_skip = skip_launch_numbers;
    return KLEOS_OK;
}

extern "C" int kleos_debug_map_hip_error(int hip_error) {
    KLEOS_HIP(static_cast<hipError_t>(hip_error));
    return KLEOS_OK;
}

// The matrix-instruction probe keeps 16 MB of operand patterns and its timing events on the current
// device until the process ends (a measurement aid: nothing of the layer touches them).
extern "C" int kleos_debug_mfma_probe(int tile, uint32_t iterations, int zero_operands, float* ms, double* flop) {
    static std::mutex mu;
    static uint32_t* data = nullptr;
    static float* sink = nullptr;
    static int filled_zero = -1, cus = 0;
    static hipEvent_t ev[2];
    if (!ms || !flop) return fail(KLEOS_EINVAL, "kleos_debug_mfma_probe: null argument");
    if ((tile != 16 && tile != 32) || iterations == 0)
        return fail(KLEOS_EINVAL, "kleos_debug_mfma_probe: tile must be 16 or 32 and iterations positive");
    std::lock_guard<std::mutex> lock(mu);
    if (!data) {
        int dev = 0;
        hipDeviceProp_t prop;
        KLEOS_HIP(hipGetDevice(&dev));
        KLEOS_HIP(hipGetDeviceProperties(&prop, dev));
        cus = prop.multiProcessorCount;
        KLEOS_HIP(hipMalloc(&sink, sizeof(float)));
        KLEOS_HIP(hipEventCreate(&ev[0]));
        KLEOS_HIP(hipEventCreate(&ev[1]));
        KLEOS_HIP(hipMalloc(&data, kMfmaProbeWords * sizeof(uint32_t)));
    }
    if (filled_zero != (zero_operands != 0)) {
        KLEOS_HIP(launch_mfma_probe_fill(data, kMfmaProbeWords, zero_operands != 0, nullptr));
        filled_zero = zero_operands != 0;
    }
    KLEOS_HIP(hipEventRecord(ev[0], nullptr));
    KLEOS_HIP(launch_mfma_probe(tile, iterations, data, sink, cus, flop, nullptr));
    KLEOS_HIP(hipEventRecord(ev[1], nullptr));
    KLEOS_HIP(hipEventSynchronize(ev[1]));
    KLEOS_HIP(hipEventElapsedTime(ms, ev[0], ev[1]));
    return KLEOS_OK;
}

extern "C" int kleos_initialize_cfg(const kleos_config_t* user_cfg) {
    if (!user_cfg) return fail(KLEOS_EINVAL, "kleos_initialize_cfg: null config");
    if (g_ctx) return fail(KLEOS_ESTATE, "Already Initialized");   // bootstrap.cuh:537
    kleos_config_t cfg = *user_cfg;
    if (int rc = kleos_config_derive(&cfg)) return rc;
    if (const char* why = unsupported_reason(cfg.E, cfg.k)) return fail(KLEOS_EUNSUPPORTED, "%s", why);

    Context* c = new Context();
    c->cfg = cfg;
    auto bail = [&](int rc) {
        if (c->arena) (void)hipFree(c->arena);
        if (c->stream) (void)hipStreamDestroy(c->stream);
        delete c;
        return rc;
    };
#define KLEOS_HIP_BAIL(expr)                                                                    \
    do {                                                                                        \
        hipError_t e_ = (expr);                                                                 \
        if (e_ != hipSuccess)                                                                   \
            return bail(fail(KLEOS_EHIP, "<%s:%d> %s:\n    %s: %s", __FILE__, __LINE__, #expr,  \
                             hipGetErrorName(e_), hipGetErrorString(e_)));                      \
    } while (0)
    KLEOS_HIP_BAIL(hipGetDevice(&c->device));
    {
        // the address of this device's static scratch, for kleos_moe_forward_static_scratch
        DeviceSetup* dev = nullptr;
        if (int rc = device_setup(&dev)) return bail(rc);
    }
    hipDeviceProp_t prop;
    KLEOS_HIP_BAIL(hipGetDeviceProperties(&prop, c->device));
    c->num_cus = prop.multiProcessorCount;
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return bail(fail(KLEOS_EUNSUPPORTED, "device '%s' is not gfx950: this library is built for MI355X only",
                         prop.gcnArchName));
    // default priority, non-blocking: the analogue of the reference's cudaStreamPerThread (types.cuh:1013)
    KLEOS_HIP_BAIL(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));

    LayerParams& p = c->base;
    params_from_config(p, cfg);
    p.gate_splits = gate_splits_for(cfg.S, cfg.H, cfg.E, cfg.PX, int(cfg.torch_dtype), c->num_cus);
    if (size_t(p.gate_splits) * cfg.S * cfg.PX * 4 >= (size_t(1) << 31))
        return bail(fail(KLEOS_EUNSUPPORTED, "the gate's partial sums (%u ranges x %u tokens x %u experts) exceed 2 GiB", p.gate_splits,
                         cfg.S, cfg.PX));
    const ArenaLayout L = layout_arena(cfg, p.n_gate_tiles, p.n_super, p.gate_splits);
    KLEOS_HIP_BAIL(hipMalloc(reinterpret_cast<void**>(&c->arena), L.total));
    c->arena_bytes = L.total;
    c->zero_begin = L.zero_begin;
    c->zero_end = L.zero_end;
    KLEOS_HIP_BAIL(hipMemsetAsync(c->arena + L.zero_begin, 0, L.zero_end - L.zero_begin, c->stream));
    KLEOS_HIP_BAIL(hipStreamSynchronize(c->stream));
    params_from_arena(p, c->arena, L);
    if (cfg.E == 1) {
        c->dense_wg = c->arena + L.dense_wg;
        c->dense_gate_out = c->arena + L.dense_gate_out;
        KLEOS_HIP_BAIL(hipMemsetAsync(c->dense_wg, 0, size_t(cfg.PX) * cfg.H * cfg.elem_bytes, c->stream));
        KLEOS_HIP_BAIL(hipStreamSynchronize(c->stream));
    }
    KLEOS_HIP_BAIL(plan_fused(p, int(cfg.torch_dtype), c->num_cus, &c->plan));
    if (c->plan.nwg > kMaxWorkgroups) return bail(fail(KLEOS_EUNSUPPORTED, "persistent grid of %u workgroups exceeds %u", c->plan.nwg, kMaxWorkgroups));
#undef KLEOS_HIP_BAIL
    g_ctx = c;
    return KLEOS_OK;
}

extern "C" int kleos_initialize(const char* config_json_path) {
    if (g_ctx) return fail(KLEOS_ESTATE, "Already Initialized");
    kleos_config_t cfg;
    if (int rc = kleos_config_parse_file(config_json_path, &cfg)) return rc;
    return kleos_initialize_cfg(&cfg);
}

extern "C" int kleos_finalize(void) {
    if (int rc = require_ctx("kleos_finalize")) return rc;
    Context* c = g_ctx;
    g_ctx = nullptr;   // bootstrap.cuh:567: isInitialized = false first
    hipError_t e1 = hipSetDevice(c->device);
    hipError_t e2 = hipStreamSynchronize(c->stream);
    hipError_t e3 = hipFree(c->arena);
    hipError_t e4 = hipStreamDestroy(c->stream);
    delete c;
    for (hipError_t e : {e1, e2, e3, e4})
        if (e != hipSuccess) return fail(KLEOS_EHIP, "kleos_finalize: %s: %s", hipGetErrorName(e), hipGetErrorString(e));
    return KLEOS_OK;
}

extern "C" int kleos_is_initialized(void) { return g_ctx != nullptr; }

extern "C" int kleos_get_rank(void) {
    if (!g_ctx) { (void)fail(KLEOS_ESTATE, "kleos_get_rank: Not initialized!"); return -1; }
    return 0;
}

extern "C" int kleos_set_device(void) {
    if (int rc = require_ctx("kleos_set_device")) return rc;
    KLEOS_HIP(hipSetDevice(g_ctx->device));
    return KLEOS_OK;
}

extern "C" int kleos_get_config(kleos_config_t* cfg) {
    if (int rc = require_ctx("kleos_get_config")) return rc;
    if (!cfg) return fail(KLEOS_EINVAL, "kleos_get_config: null argument");
    *cfg = g_ctx->cfg;
    return KLEOS_OK;
}

extern "C" int kleos_set_mode(int mode) {
    if (int rc = require_ctx("kleos_set_mode")) return rc;
    if (mode != KLEOS_MODE_FUSED && mode != KLEOS_MODE_PHASED) return fail(KLEOS_EINVAL, "kleos_set_mode: unknown mode %d", mode);
    g_ctx->mode = mode;
    return KLEOS_OK;
}

extern "C" int kleos_get_mode(void) { return g_ctx ? g_ctx->mode : -1; }

extern "C" int kleos_set_schedule(int schedule) {
    if (int rc = require_ctx("kleos_set_schedule")) return rc;
    if (schedule != KLEOS_SCHEDULE_AUTO && schedule != KLEOS_SCHEDULE_DYNAMIC && schedule != KLEOS_SCHEDULE_STATIC)
        return fail(KLEOS_EINVAL, "kleos_set_schedule: unknown schedule %d", schedule);
    g_ctx->schedule = schedule;
    return KLEOS_OK;
}

extern "C" int kleos_get_schedule(void) { return g_ctx ? g_ctx->schedule : -1; }

extern "C" int kleos_set_cooperative_launch(int on) {
    if (int rc = require_ctx("kleos_set_cooperative_launch")) return rc;
    if (on) {
        int supported = 0;
        KLEOS_HIP(hipDeviceGetAttribute(&supported, hipDeviceAttributeCooperativeLaunch, g_ctx->device));
        if (!supported) return fail(KLEOS_EUNSUPPORTED, "kleos_set_cooperative_launch: the device does not support cooperative launches");
    }
    g_ctx->plan.cooperative = on != 0;
    return KLEOS_OK;
}

extern "C" int kleos_schedule_taken(int* schedule) {
    if (int rc = require_ctx("kleos_schedule_taken")) return rc;
    if (!schedule) return fail(KLEOS_EINVAL, "kleos_schedule_taken: null argument");
    Context& c = *g_ctx;
    if (c.fused_seq == 0) return fail(KLEOS_ESTATE, "kleos_schedule_taken: no persistent launch yet");
    KLEOS_HIP(hipSetDevice(c.device));
    KLEOS_HIP(hipStreamSynchronize(c.stream));
    unsigned long long flag = 0;   // workgroup 0, word 14 of its stamp row
    KLEOS_HIP(hipMemcpy(&flag, c.base.stamps + 14, sizeof(flag), hipMemcpyDeviceToHost));
    *schedule = flag ? KLEOS_SCHEDULE_STATIC : KLEOS_SCHEDULE_DYNAMIC;
    return KLEOS_OK;
}

extern "C" int kleos_moe_forward(const void* iP, void* oP) {
    if (int rc = require_ctx("kleos_moe_forward")) return rc;
    KLEOS_HIP(hipSetDevice(g_ctx->device));   // moe.cuh:192
    return enqueue_forward(*g_ctx, iP, oP, nullptr);
}

extern "C" int kleos_moe_forward_dense(const void* iP, void* oP) {
    if (int rc = require_ctx("kleos_moe_forward_dense")) return rc;
    Context& c = *g_ctx;
    if (c.cfg.E != 1) return fail(KLEOS_ESTATE, "kleos_moe_forward_dense: the context holds %u experts; the dense packing is for num_experts 1", c.cfg.E);
    // the bias block D1 must leave D2 16-byte aligned for the kernels' 16-byte loads
    if ((size_t(c.cfg.I) * c.cfg.elem_bytes) & 15u)
        return fail(KLEOS_EUNSUPPORTED, "kleos_moe_forward_dense: intermediate_size * sizeof(Element) must be a multiple of 16");
    KLEOS_HIP(hipSetDevice(c.device));
    return enqueue_forward(c, iP, oP, nullptr, true);
}

extern "C" int kleos_moe_forward_bench(const void* iP, void* oP, uint32_t skip, uint32_t trials,
                                       float* ms_per_launch) {
    if (int rc = require_ctx("kleos_moe_forward_bench")) return rc;
    if (!ms_per_launch || trials == 0) return fail(KLEOS_EINVAL, "kleos_moe_forward_bench: need trials > 0 and a result pointer");
    Context& c = *g_ctx;
    KLEOS_HIP(hipSetDevice(c.device));
    for (uint32_t i = 0; i < skip; ++i)
        if (int rc = enqueue_forward(c, iP, oP, nullptr)) return rc;
    const bool phased = c.mode == KLEOS_MODE_PHASED;
    hipEvent_t start, stop;
    KLEOS_HIP(hipEventCreate(&start));
    KLEOS_HIP(hipEventCreate(&stop));
    std::vector<hipEvent_t> ev;
    if (phased) {
        ev.resize(size_t(trials) * 6);
        for (auto& e : ev) KLEOS_HIP(hipEventCreate(&e));
    }
    int rc = KLEOS_OK;
    KLEOS_HIP(hipEventRecord(start, c.stream));                       // moe.cuh:166
    for (uint32_t i = 0; i < trials && rc == KLEOS_OK; ++i)
        rc = enqueue_forward(c, iP, oP, phased ? &ev[size_t(i) * 6] : nullptr);
    if (rc == KLEOS_OK) {
        KLEOS_HIP(hipEventRecord(stop, c.stream));                    // moe.cuh:178
        KLEOS_HIP(hipStreamSynchronize(c.stream));
        float ms = 0.f;
        KLEOS_HIP(hipEventElapsedTime(&ms, start, stop));
        *ms_per_launch = ms / float(trials);                          // moe.cuh:181
        for (float& v : c.phase_ms) v = 0.f;
        if (!phased) {
            // phase boundaries of the last launch, stamped by every workgroup of the persistent kernel
            std::vector<unsigned long long> st(size_t(c.plan.nwg) * 16);
            KLEOS_HIP(hipMemcpy(st.data(), c.base.stamps, st.size() * 8, hipMemcpyDeviceToHost));
            unsigned long long t0 = ~0ull, b[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int i = 0; i < 6; ++i) c.sched_stats[i] = 0.0;
            for (uint32_t w = 0; w < c.plan.nwg; ++w) {
                t0 = std::min(t0, st[size_t(w) * 16]);
                for (int i = 0; i < 8; ++i) b[i] = std::max(b[i], st[size_t(w) * 16 + i]);
                for (int i = 0; i < 6; ++i) c.sched_stats[i] += double(st[size_t(w) * 16 + 8 + i]);
            }
            for (int i = 0; i < 3; ++i) c.sched_stats[i] *= 1e-5 / double(c.plan.nwg);   // mean ms per workgroup
            const float tick_ms = 1e-5f;   // 100 MHz
            c.phase_ms[0] = float(b[2] - t0) * tick_ms;        // gate, through the first grid barrier
            c.phase_ms[1] = float(b[4] - b[2]) * tick_ms;      // slots, through the second
            c.phase_ms[2] = float(b[6] - b[4]) * tick_ms;      // both projections, through the third
            c.phase_ms[3] = 0.f;
            c.phase_ms[4] = float(b[7] - b[6]) * tick_ms;      // combine
        }
        if (phased) {
            for (uint32_t i = 0; i < trials; ++i)
                for (int ph = 0; ph < 5; ++ph) {
                    float t = 0.f;
                    KLEOS_HIP(hipEventElapsedTime(&t, ev[size_t(i) * 6 + ph], ev[size_t(i) * 6 + ph + 1]));
                    c.phase_ms[ph] += t / float(trials);
                }
        }
    } else {
        (void)hipStreamSynchronize(c.stream);
    }
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    for (auto& e : ev) (void)hipEventDestroy(e);
    if (rc == KLEOS_OK) rc = check_scheduler(c);
    return rc;
}

extern "C" int kleos_stream_synchronize(void) {
    if (int rc = require_ctx("kleos_stream_synchronize")) return rc;
    KLEOS_HIP(hipStreamSynchronize(g_ctx->stream));
    return check_scheduler(*g_ctx);
}

extern "C" void* kleos_stream(void) { return g_ctx ? static_cast<void*>(g_ctx->stream) : nullptr; }

extern "C" int kleos_moe_debug_views(kleos_debug_views_t* v) {
    if (int rc = require_ctx("kleos_moe_debug_views")) return rc;
    if (!v) return fail(KLEOS_EINVAL, "kleos_moe_debug_views: null argument");
    const LayerParams& p = g_ctx->base;
    v->logits = p.logits;
    v->topk_expert = p.topk_expert;
    v->topk_prob = p.topk_prob;
    v->combine_den = p.combine_den;
    v->topk_slot = p.topk_slot;
    v->expert_count = p.expert_count;
    v->slot_token = p.slot_token;
    return KLEOS_OK;
}

extern "C" int kleos_debug_copy_to_host(void* host_dst, const void* device_src, size_t bytes) {
    if (int rc = require_ctx("kleos_debug_copy_to_host")) return rc;
    if (!host_dst || !device_src) return fail(KLEOS_EINVAL, "kleos_debug_copy_to_host: null argument");
    KLEOS_HIP(hipStreamSynchronize(g_ctx->stream));
    KLEOS_HIP(hipMemcpy(host_dst, device_src, bytes, hipMemcpyDeviceToHost));
    return KLEOS_OK;
}

extern "C" int kleos_scheduler_stats(double stats[6]) {
    if (int rc = require_ctx("kleos_scheduler_stats")) return rc;
    if (!stats) return fail(KLEOS_EINVAL, "kleos_scheduler_stats: null argument");
    for (int i = 0; i < 6; ++i) stats[i] = g_ctx->sched_stats[i];
    return KLEOS_OK;
}

extern "C" int kleos_measure_throughput(uint32_t trials, float* median_ms, float* throughput) {
    return kleos_measure_throughput_output(trials, median_ms, throughput, nullptr, 0);
}

extern "C" int kleos_measure_throughput_output(uint32_t trials, float* median_ms, float* throughput, void* y_host,
                                               size_t y_bytes) {
    if (int rc = require_ctx("kleos_measure_throughput")) return rc;
    if (!median_ms || !throughput || trials == 0 || trials > 1024)
        return fail(KLEOS_EINVAL, "kleos_measure_throughput: need result pointers and 1 <= trials <= 1024");
    Context& c = *g_ctx;
    if (y_bytes && !y_host) return fail(KLEOS_EINVAL, "kleos_measure_throughput_output: null result buffer");
    if (y_bytes > size_t(c.cfg.pEC) * c.cfg.H * c.cfg.elem_bytes)
        return fail(KLEOS_EINVAL, "kleos_measure_throughput_output: the probe's result holds %zu bytes",
                    size_t(c.cfg.pEC) * c.cfg.H * c.cfg.elem_bytes);
    KLEOS_HIP(hipSetDevice(c.device));
    // One expert at full padded capacity, as the reference's probe (throughput.cuh:104-170):
    // M = pEC rows, up-projection to I columns over K = H, activation, down-projection back to H.
    const kleos_config_t& cfg = c.cfg;
    const size_t eb = cfg.elem_bytes, M = cfg.pEC, H = cfg.H, I = cfg.I;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
    const size_t o_x = take(M * H * eb), o_wu = take(I * H * eb), o_wd = take(H * I * eb), o_bu = take(I * eb),
                 o_bd = take(H * eb), o_h1 = take(M * I * eb), o_y = take(y_expert_elems(uint32_t(M), cfg.H, cfg.elem_bytes) * eb), o_cnt = take(4),
                 o_tok = take(M * 4);
    char* buf = nullptr;
    KLEOS_HIP(hipMalloc(reinterpret_cast<void**>(&buf), off));
    int rc = KLEOS_OK;
    std::vector<hipEvent_t> ev(size_t(trials) * 2, nullptr);
    auto body = [&]() -> int {
        // finite, small operands (every byte 0x3c: 0.0115 in bf16 and fp32, 1.06 in fp16); the
        // timing does not depend on the values
        KLEOS_HIP(hipMemsetAsync(buf, 0x3c, o_cnt, c.stream));
        std::vector<int32_t> tok(M);
        for (size_t i = 0; i < M; ++i) tok[i] = int32_t(i);
        const uint32_t count = uint32_t(M);
        KLEOS_HIP(hipMemcpyAsync(buf + o_cnt, &count, 4, hipMemcpyHostToDevice, c.stream));
        KLEOS_HIP(hipMemcpyAsync(buf + o_tok, tok.data(), M * 4, hipMemcpyHostToDevice, c.stream));
        KLEOS_HIP(hipStreamSynchronize(c.stream));
        LayerParams q{};
        q.S = uint32_t(M); q.H = cfg.H; q.I = cfg.I; q.E = 1; q.k = 1; q.PX = 64; q.EC = uint32_t(M);
        q.cap_rows = uint32_t(M); q.act = cfg.hidden_act;
        q.x = buf + o_x; q.w_up = buf + o_wu; q.w_down = buf + o_wd; q.b_up = buf + o_bu; q.b_down = buf + o_bd;
        q.h1 = buf + o_h1; q.y = buf + o_y;
        q.expert_count = reinterpret_cast<uint32_t*>(buf + o_cnt);
        q.slot_token = reinterpret_cast<int32_t*>(buf + o_tok);
        const int dt = int(cfg.torch_dtype);
        for (auto& e : ev) KLEOS_HIP(hipEventCreate(&e));
        for (uint32_t t = 0; t < trials + 2; ++t) {          // two warm-up rounds
            const bool timed = t >= 2;
            if (timed) KLEOS_HIP(hipEventRecord(ev[size_t(t - 2) * 2], c.stream));
            KLEOS_HIP(launch_expert_gemm(q, dt, 0, c.num_cus, c.stream));
            KLEOS_HIP(launch_expert_gemm(q, dt, 1, c.num_cus, c.stream));
            if (timed) KLEOS_HIP(hipEventRecord(ev[size_t(t - 2) * 2 + 1], c.stream));
        }
        KLEOS_HIP(hipStreamSynchronize(c.stream));
        std::vector<float> ms(trials);
        for (uint32_t t = 0; t < trials; ++t) KLEOS_HIP(hipEventElapsedTime(&ms[t], ev[size_t(t) * 2], ev[size_t(t) * 2 + 1]));
        std::sort(ms.begin(), ms.end());
        *median_ms = ms[trials / 2];                          // throughput.cuh:166 (findMedian)
        *throughput = *median_ms > 0.f ? 1.0f / *median_ms : 0.f;
        if (y_bytes) {
            // the caller gets y[pEC, H] row by row, whatever the layout the kernels keep it in
            std::vector<char> dev_y(y_expert_elems(uint32_t(M), cfg.H, cfg.elem_bytes) * eb), rows(M * H * eb);
            KLEOS_HIP(hipMemcpy(dev_y.data(), buf + o_y, dev_y.size(), hipMemcpyDeviceToHost));
            for (size_t m = 0; m < M; ++m)
                for (size_t n = 0; n < H; ++n)
                    std::memcpy(&rows[(m * H + n) * eb], &dev_y[y_offset(0, uint32_t(m), uint32_t(n), uint32_t(M), cfg.H, cfg.elem_bytes) * eb], eb);
            std::memcpy(y_host, rows.data(), y_bytes);
        }
        return KLEOS_OK;
    };
    rc = body();
    (void)hipStreamSynchronize(c.stream);
    for (auto& e : ev) if (e) (void)hipEventDestroy(e);
    (void)hipFree(buf);
    return rc;
}

extern "C" int kleos_debug_set_wait_ticks(unsigned long long ticks) {
    if (int rc = require_ctx("kleos_debug_set_wait_ticks")) return rc;
    g_ctx->base.wait_ticks = ticks ? ticks : kDefaultWaitTicks;
    return KLEOS_OK;
}

extern "C" int kleos_debug_skip_launch_number(void) {
    if (int rc = require_ctx("kleos_debug_skip_launch_number")) return rc;
    g_ctx->fused_seq++;
    return KLEOS_OK;
}

extern "C" int kleos_gate_loss(float* loss, float* mean_prob, float* mean_count) {
    if (int rc = require_ctx("kleos_gate_loss")) return rc;
    Context& c = *g_ctx;
    if (!c.cfg.is_training) return fail(KLEOS_ESTATE, "kleos_gate_loss: the context was initialised with is_training 0");
    if (!loss) return fail(KLEOS_EINVAL, "kleos_gate_loss: null argument");
    KLEOS_HIP(hipSetDevice(c.device));
    KLEOS_HIP(hipStreamSynchronize(c.stream));
    const size_t E = c.cfg.E;
    KLEOS_HIP(hipMemcpy(loss, c.base.gate_loss + 2 * E, 4, hipMemcpyDeviceToHost));
    if (mean_prob) KLEOS_HIP(hipMemcpy(mean_prob, c.base.gate_loss, E * 4, hipMemcpyDeviceToHost));
    if (mean_count) KLEOS_HIP(hipMemcpy(mean_count, c.base.gate_loss + E, E * 4, hipMemcpyDeviceToHost));
    return check_scheduler(c);
}

extern "C" int kleos_phase_stamps(unsigned long long* stamps, uint32_t max_workgroups, uint32_t* n_workgroups) {
    if (int rc = require_ctx("kleos_phase_stamps")) return rc;
    if (!stamps || !n_workgroups) return fail(KLEOS_EINVAL, "kleos_phase_stamps: null argument");
    Context& c = *g_ctx;
    KLEOS_HIP(hipSetDevice(c.device));
    KLEOS_HIP(hipStreamSynchronize(c.stream));
    *n_workgroups = c.plan.nwg;
    const uint32_t n = std::min(c.plan.nwg, max_workgroups);
    std::vector<unsigned long long> st(size_t(n) * 16);
    if (n) KLEOS_HIP(hipMemcpy(st.data(), c.base.stamps, st.size() * 8, hipMemcpyDeviceToHost));
    for (uint32_t w = 0; w < n; ++w)
        for (int i = 0; i < 8; ++i) stamps[size_t(w) * 8 + i] = st[size_t(w) * 16 + i];
    return KLEOS_OK;
}

extern "C" int kleos_phase_times(float ms[5]) {
    if (int rc = require_ctx("kleos_phase_times")) return rc;
    if (!ms) return fail(KLEOS_EINVAL, "kleos_phase_times: null argument");
    for (int i = 0; i < 5; ++i) ms[i] = g_ctx->phase_ms[i];
    return KLEOS_OK;
}
