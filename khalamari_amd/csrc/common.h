// Error reporting and small helpers shared by the host sources of the C ABI.
#pragma once
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "../../include/khm_gqa_sdpa.h"

namespace khm {

std::string& last_error_storage();

inline int fail(int status, const char* format, ...) {
    char buffer[512];
    va_list args;
    va_start(args, format);
    vsnprintf(buffer, sizeof buffer, format, args);
    va_end(args);
    last_error_storage() = buffer;
    return status;
}

inline void clear_error() { last_error_storage().clear(); }

// The reference asserts; the C ABI reports the same condition as an error code.
#define KHM_REQUIRE(condition, ...)                                        \
    do {                                                                   \
        if (!(condition)) return ::khm::fail(KHM_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

// A kernel launch whose status the caller reads with hipGetLastError() afterwards.  The runtime keeps a thread's last error
// until somebody reads it, whoever caused it (a failed copy or query of the host program's, say; without this, a launch
// after such a call was reported as "launch failed: invalid argument"): it is read away first, so that the check after
// the launch reports this launch and nothing older.  (Expands only in sources that include the HIP runtime header.)
#define KHM_LAUNCH(...)                  \
    do {                                 \
        (void)hipGetLastError();         \
        hipLaunchKernelGGL(__VA_ARGS__); \
    } while (0)

inline uint32_t div_ceil_u32(uint32_t a, uint32_t b) { return a / b + (a % b != 0); }
inline uint64_t div_ceil_u64(uint64_t a, uint64_t b) { return a / b + (a % b != 0); }

inline bool is_power_of_two(uint32_t v) { return v != 0 && (v & (v - 1)) == 0; }

// Smallest power of two >= v (2^31 for anything above it: the callers clamp long before that).
inline uint32_t next_power_of_two(uint32_t v) {
    uint32_t p = 1;
    while (p < v && p < 0x80000000u) p <<= 1;
    return p;
}

inline uint32_t ilog2_u64(uint64_t v) {
    uint32_t r = 0;
    while (v >>= 1) ++r;
    return r;
}

inline uint32_t kv_element_bytes(uint32_t kv_dtype) { return kv_dtype == KHM_DTYPE_FP8_E4M3FN ? 1u : 2u; }
inline uint32_t dtype_item_size(uint32_t dtype) {
    switch (dtype) {
        case KHM_DTYPE_F32: return 4;
        case KHM_DTYPE_BF16: return 2;
        case KHM_DTYPE_FP8_E4M3FN: return 1;
        case KHM_DTYPE_U32: return 4;
        default: return 0;
    }
}

// sdpa::Config::validate (components/gqa/sdpa.rs:229-237).
int validate_sdpa_config(const khm_sdpa_config* config);
// ExecutionVariant::supports (sdpa.rs:162-215).
bool variant_supports(const khm_sdpa_variant& variant, const khm_sdpa_config& config);
// Which gfx950 Map kernel family serves a variant: 0 = none, 1 = small-tile split-KV kernel
// (<= 64 Q coordinates per block), 2 = tiled prefill kernel.
int kernel_family(const khm_sdpa_config& config, const khm_sdpa_variant& variant, uint32_t kv_dtype, std::string* why);

}  // namespace khm
