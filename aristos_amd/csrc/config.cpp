// Run-time reader of kleos_config.json and the derived layer constants.
//
// The reference turns the JSON into -D macros at CMake configure time (csrc/CMakeLists.txt:186-252)
// and derives every size in the compile-time struct ACC (csrc/include/kleos/types.cuh:442-513).
// Here the same keys are read at run time and the same formulas are evaluated on the host.
#include "common.hpp"

#include <algorithm>
#include <cctype>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

namespace kleos_amd {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

namespace {

// A flat JSON object of "key": number pairs is all the schema allows; anything else is rejected.
struct FlatJson {
    const char* p;
    explicit FlatJson(const char* s) : p(s) {}
    void ws() { while (*p && std::isspace(static_cast<unsigned char>(*p))) ++p; }
    bool key(std::string& out) {
        ws();
        if (*p != '"') return false;
        ++p;
        out.clear();
        while (*p && *p != '"') {
            if (*p == '\\') return false;  // no escapes in schema keys
            out.push_back(*p++);
        }
        if (*p != '"') return false;
        ++p;
        return true;
    }
    bool number(double& out) {
        ws();
        char* end = nullptr;
        errno = 0;
        out = std::strtod(p, &end);
        if (end == p || errno == ERANGE) return false;
        p = end;
        return true;
    }
};

struct KeySlot {
    const char* name;
    bool required;      // csrc/kleos_config.schema.json:73-88
    bool is_real;
    size_t offset;
};

#define KSLOT(field, req, real) {#field, req, real, offsetof(kleos_config_t, field)}
const KeySlot kSlots[] = {
    KSLOT(capacity_factor, true, true),
    KSLOT(drop_tokens, true, false),
    KSLOT(expert_top_k, true, false),
    KSLOT(global_batch, false, false),
    KSLOT(is_training, true, false),
    KSLOT(hidden_act, true, false),
    KSLOT(hidden_size, true, false),
    KSLOT(intermediate_size, true, false),
    KSLOT(mini_batch, true, false),
    KSLOT(moe_frequency, true, false),
    KSLOT(num_experts, true, false),
    KSLOT(num_layers, true, false),
    KSLOT(sequence_len, true, false),
    KSLOT(torch_dtype, true, false),
    KSLOT(vocab_size, true, false),
};
#undef KSLOT
constexpr int kNumSlots = sizeof(kSlots) / sizeof(kSlots[0]);

inline uint64_t ceil_div(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

}  // namespace
}  // namespace kleos_amd

using namespace kleos_amd;

extern "C" void kleos_config_defaults(kleos_config_t* cfg) {
    if (!cfg) return;
    std::memset(cfg, 0, sizeof *cfg);
    cfg->capacity_factor = 1.0;
    cfg->drop_tokens = 1;
    cfg->expert_top_k = 2;
    cfg->global_batch = 256;
    cfg->is_training = 0;
    cfg->hidden_act = KLEOS_ACT_RELU;
    cfg->hidden_size = 2048;
    cfg->intermediate_size = 2048;
    cfg->mini_batch = 1;
    cfg->moe_frequency = 1;
    cfg->num_experts = 64;
    cfg->num_layers = 1;
    cfg->sequence_len = 8192;
    cfg->torch_dtype = KLEOS_DTYPE_BF16;
    cfg->vocab_size = 32000;
}

extern "C" int kleos_config_parse_string(const char* text, kleos_config_t* cfg) {
    if (!text || !cfg) return fail(KLEOS_EINVAL, "kleos_config_parse_string: null argument");
    std::memset(cfg, 0, sizeof *cfg);
    bool seen[kNumSlots] = {};
    FlatJson js(text);
    js.ws();
    if (*js.p != '{') return fail(KLEOS_EPARSE, "config: expected '{' at offset %ld", long(js.p - text));
    ++js.p;
    js.ws();
    if (*js.p == '}') {
        ++js.p;
    } else {
        for (;;) {
            std::string key;
            if (!js.key(key)) return fail(KLEOS_EPARSE, "config: expected a quoted key at offset %ld", long(js.p - text));
            js.ws();
            if (*js.p != ':') return fail(KLEOS_EPARSE, "config: expected ':' after key '%s'", key.c_str());
            ++js.p;
            double v = 0;
            if (!js.number(v)) return fail(KLEOS_EPARSE, "config: key '%s' needs a numeric value", key.c_str());
            int hit = -1;
            for (int i = 0; i < kNumSlots; ++i)
                if (key == kSlots[i].name) hit = i;
            if (hit >= 0) {
                if (seen[hit]) return fail(KLEOS_EPARSE, "config: key '%s' given twice", key.c_str());
                seen[hit] = true;
                char* base = reinterpret_cast<char*>(cfg);
                if (kSlots[hit].is_real) {
                    *reinterpret_cast<double*>(base + kSlots[hit].offset) = v;
                } else {
                    if (v < 0 || v > 4294967295.0 || v != std::floor(v))
                        return fail(KLEOS_EPARSE, "config: key '%s' must be a non-negative integer, got %g", key.c_str(), v);
                    *reinterpret_cast<uint32_t*>(base + kSlots[hit].offset) = static_cast<uint32_t>(v);
                }
            }
            // unknown keys are ignored: the schema does not set additionalProperties: false
            js.ws();
            if (*js.p == ',') { ++js.p; continue; }
            if (*js.p == '}') { ++js.p; break; }
            return fail(KLEOS_EPARSE, "config: expected ',' or '}' at offset %ld", long(js.p - text));
        }
    }
    js.ws();
    if (*js.p) return fail(KLEOS_EPARSE, "config: trailing characters after the object");
    for (int i = 0; i < kNumSlots; ++i)
        if (kSlots[i].required && !seen[i])
            return fail(KLEOS_EPARSE, "config: required key '%s' is missing", kSlots[i].name);
    if (!seen[3]) cfg->global_batch = 0;
    return KLEOS_OK;
}

extern "C" int kleos_config_parse_file(const char* path, kleos_config_t* cfg) {
    if (!path || !cfg) return fail(KLEOS_EINVAL, "kleos_config_parse_file: null argument");
    FILE* f = std::fopen(path, "rb");
    if (!f) return fail(KLEOS_EIO, "config: cannot open '%s': %s", path, std::strerror(errno));
    std::string text;
    char buf[4096];
    size_t n;
    while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, n);
    std::fclose(f);
    return kleos_config_parse_string(text.c_str(), cfg);
}

extern "C" int kleos_config_derive(kleos_config_t* c) {
    if (!c) return fail(KLEOS_EINVAL, "kleos_config_derive: null argument");
    if (c->drop_tokens > 1) return fail(KLEOS_EINVAL, "drop_tokens must be 0 or 1, got %u", c->drop_tokens);
    if (c->is_training > 1) return fail(KLEOS_EINVAL, "is_training must be 0 or 1, got %u", c->is_training);
    if (c->hidden_act > KLEOS_ACT_GELU) return fail(KLEOS_EINVAL, "hidden_act must be 0 (relu) or 1 (gelu), got %u", c->hidden_act);
    if (c->torch_dtype > KLEOS_DTYPE_FP16) return fail(KLEOS_EINVAL, "torch_dtype must be 0..3, got %u", c->torch_dtype);
    if (c->num_experts < 1) return fail(KLEOS_EINVAL, "num_experts must be >= 1");
    if (c->num_experts > 65535) return fail(KLEOS_EINVAL, "num_experts must be <= 65535 (types.cuh:479), got %u", c->num_experts);
    if (c->expert_top_k < 1) return fail(KLEOS_EINVAL, "expert_top_k must be >= 1");
    if (c->expert_top_k > c->num_experts)
        return fail(KLEOS_EINVAL, "expert_top_k (%u) must be <= num_experts (%u) (types.cuh:497)", c->expert_top_k, c->num_experts);
    if (!(c->capacity_factor >= 1.0) || !std::isfinite(c->capacity_factor))
        return fail(KLEOS_EINVAL, "capacity_factor must be a finite value >= 1 (schema minimum), got %g", c->capacity_factor);
    if (c->mini_batch < 1 || c->sequence_len < 1) return fail(KLEOS_EINVAL, "sequence_len and mini_batch must be >= 1");
    const uint64_t S = uint64_t(c->sequence_len) * c->mini_batch;                       // types.cuh:471
    if (S % 128) return fail(KLEOS_EINVAL, "sequence_len*mini_batch (%llu) must be a multiple of 128 (bootstrap.cuh:542)", (unsigned long long)S);
    if (S > (1u << 30)) return fail(KLEOS_EINVAL, "sequence_len*mini_batch (%llu) is too large", (unsigned long long)S);
    if (c->hidden_size == 0 || c->hidden_size % 64)
        return fail(KLEOS_EINVAL, "hidden_size (%u) must be a positive multiple of 64 (bootstrap.cuh:543)", c->hidden_size);
    if (c->intermediate_size == 0 || c->intermediate_size % 64)
        return fail(KLEOS_EINVAL, "intermediate_size (%u) must be a positive multiple of 64 (bootstrap.cuh:543)", c->intermediate_size);

    c->S = uint32_t(S);
    c->H = c->hidden_size;
    c->I = c->intermediate_size;                                                        // types.cuh:472
    c->E = c->num_experts;
    c->k = c->expert_top_k;
    c->PX = uint32_t(ceil_div(c->E, 64) * 64);                                          // types.cuh:481
    // types.cuh:498-499: EC = (drop ? ceil(S/E) : S) * CF * TK. A real-valued capacity factor is
    // rounded up, which reproduces the reference for every integer factor.
    const double base = c->drop_tokens ? double(ceil_div(S, c->E)) : double(S);
    const double ec = std::ceil(base * c->capacity_factor * double(c->k) - 1e-9);
    if (ec > 4.0e9) return fail(KLEOS_EINVAL, "expert capacity overflows 32 bits");
    c->EC = uint32_t(ec);
    c->pEC = uint32_t(ceil_div(c->EC, 128) * 128);                                      // types.cuh:500
    c->cap_rows = uint32_t(std::min<uint64_t>(c->pEC, S));
    c->elem_bytes = (c->torch_dtype == KLEOS_DTYPE_FP32 || c->torch_dtype == KLEOS_DTYPE_TF32) ? 4u : 2u;
    // Packed buffers: moe.cuh:92-98, main.cu:23-30.
    const uint64_t H = c->H, I = c->I, E = c->E, PX = c->PX;
    c->off_x = 0;
    c->off_gate_w = S * H;
    c->off_w_up = c->off_gate_w + PX * H;
    c->off_w_down = c->off_w_up + E * I * H;
    c->off_b_up = c->off_w_down + E * H * I;
    c->off_b_down = c->off_b_up + E * I;
    c->in_elems = c->off_b_down + E * H;
    c->off_gate_out = 0;
    c->off_moe_out = S * PX;
    c->out_elems = c->off_moe_out + S * H;
    return KLEOS_OK;
}

extern "C" const char* kleos_last_error(void) { return g_last_error.c_str(); }
