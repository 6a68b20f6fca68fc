// Static capability of the GQA SDPA component: which (kind, tile, stage) variants are legal for a
// head geometry.  Behaviour follows crates/inference-backend-metal/src/components/gqa/sdpa.rs:
// ExecutionVariant::{sliced_kv, sliced_q, supports} (:60-215), Config::validate (:229-237) and
// Registry::new (:248-267, helpers :304-336).  `required_threads` keeps the reference's unit
// (32 lanes per SIMDgroup) so executor-side policies that read it keep their meaning; the gfx950
// launch width is chosen by the launcher.
#include <vector>

#include "common.h"

namespace khm {

int validate_sdpa_config(const khm_sdpa_config* config) {
    KHM_REQUIRE(config != nullptr, "GQA SDPA config must not be null");
    KHM_REQUIRE(config->io_dtype == KHM_DTYPE_F32 || config->io_dtype == KHM_DTYPE_BF16,
                "GQA SDPA io dtype must be Float32 or Bfloat16");
    KHM_REQUIRE(config->num_q_heads > 0, "GQA SDPA requires Q heads");
    KHM_REQUIRE(config->num_kv_heads > 0, "GQA SDPA requires KV heads");
    KHM_REQUIRE(config->num_q_heads % config->num_kv_heads == 0, "GQA Q heads must be a multiple of KV heads");
    KHM_REQUIRE(config->head_dim > 0, "GQA SDPA requires a head dimension");
    KHM_REQUIRE(config->tokens_per_page > 0, "GQA SDPA requires tokens per page");
    return KHM_OK;
}

static uint32_t q_heads_per_kv_head(const khm_sdpa_config& config) { return config.num_q_heads / config.num_kv_heads; }

static bool sliced_q_profile(uint32_t head_dim, uint32_t tokens_per_page) {
    return (head_dim == 128 && (tokens_per_page == 8 || tokens_per_page == 16)) ||
           (head_dim == 256 && (tokens_per_page == 8 || tokens_per_page == 16 || tokens_per_page == 32));
}

// Number of 8-coordinate SIMDgroups the reference assigns to a sliced-Q tile (sdpa.rs:103-123);
// false when the product overflows u32.
static bool sliced_q_simdgroups(uint32_t kind, uint32_t max_q_tokens, uint32_t max_q_heads, uint64_t* groups) {
    uint64_t count = 0;
    switch (kind) {
        case KHM_MAP_Q_TOKENS_PER_HEAD: count = (uint64_t)div_ceil_u32(max_q_tokens, 8) * max_q_heads; break;
        case KHM_MAP_Q_HEADS_PER_TOKEN: count = (uint64_t)div_ceil_u32(max_q_heads, 8) * max_q_tokens; break;
        case KHM_MAP_Q_TOKENS_AND_HEADS: count = div_ceil_u64((uint64_t)max_q_tokens * max_q_heads, 8); break;
        default: return false;
    }
    if (count > 0xffffffffull / 32) return false;
    *groups = count;
    return true;
}

static void sliced_kv_reduce_shape(const khm_sdpa_config& config, uint32_t* max_q_tokens, uint32_t* max_q_heads) {
    const uint32_t coordinates = 256 / (config.head_dim < 256 ? config.head_dim : 256);
    uint32_t heads = config.num_q_heads < coordinates ? config.num_q_heads : coordinates;
    if (heads < 1) heads = 1;
    uint32_t tokens = coordinates / heads;
    if (tokens < 1) tokens = 1;
    *max_q_heads = heads;
    *max_q_tokens = tokens;
}

bool variant_supports(const khm_sdpa_variant& v, const khm_sdpa_config& config) {
    if (v.kv_cache_tokens_per_page != config.tokens_per_page || v.map_max_q_tokens == 0 || v.map_max_q_heads == 0 ||
        v.map_max_q_heads > q_heads_per_kv_head(config) || v.map_kv_tokens_per_iteration == 0 ||
        v.map_required_threads == 0 || v.reduce_max_q_tokens == 0 || v.reduce_max_q_heads == 0 ||
        v.reduce_required_threads == 0) {
        return false;
    }
    if (v.map_kind == KHM_MAP_SLICED_KV) {
        uint32_t reduce_tokens, reduce_heads;
        sliced_kv_reduce_shape(config, &reduce_tokens, &reduce_heads);
        return v.map_max_q_tokens == 1 && v.map_max_q_heads <= 8 && v.map_kv_tokens_per_iteration <= 1024 &&
               is_power_of_two(v.map_required_threads) && v.map_required_threads >= 32 &&
               v.map_required_threads <= 256 && v.reduce_max_q_tokens == reduce_tokens &&
               v.reduce_max_q_heads == reduce_heads && v.reduce_required_threads == 256;
    }
    uint64_t groups = 0;
    if (!sliced_q_simdgroups(v.map_kind, v.map_max_q_tokens, v.map_max_q_heads, &groups)) return false;
    const uint64_t expected_threads = groups * 32;
    const uint32_t t = v.map_max_q_tokens;
    const uint32_t s = v.map_kv_tokens_per_iteration;
    return config.io_dtype == KHM_DTYPE_BF16 && sliced_q_profile(config.head_dim, config.tokens_per_page) &&
           (t == 1 || t == 2 || t == 4 || t == 8 || t == 16 || t == 32) &&
           (s == 8 || s == 16 || s == 32 || s == 64 || s == 128) && v.map_required_threads == expected_threads &&
           v.map_required_threads <= 1024 && v.reduce_max_q_tokens == t && v.reduce_max_q_heads == 1 &&
           v.reduce_required_threads == v.map_required_threads;
}

int kernel_family(const khm_sdpa_config& config, const khm_sdpa_variant& variant, uint32_t kv_dtype, std::string* why) {
    auto no = [&](const char* reason) {
        if (why) *why = reason;
        return 0;
    };
    if (config.io_dtype != KHM_DTYPE_BF16) return no("gfx950 kernels are built for bf16 Q/output only");
    if (config.head_dim != 128 && config.head_dim != 256) return no("gfx950 kernels are built for head_dim 128 and 256");
    if (config.tokens_per_page != 8 && config.tokens_per_page != 16 && config.tokens_per_page != 32)
        return no("gfx950 kernels are built for 8, 16 or 32 tokens per page");
    if (kv_dtype != KHM_DTYPE_BF16 && kv_dtype != KHM_DTYPE_FP8_E4M3FN) return no("gfx950 kernels read bf16 or FP8 E4M3FN K/V pages");
    const uint64_t coordinates = (uint64_t)variant.map_max_q_tokens * variant.map_max_q_heads;
    // one 16-column MFMA tile: the split-KV kernel (waves share nothing); wider tiles share K/V through LDS.  Both
    // kernel families read bf16 and FP8 E4M3FN pages.
    if (coordinates <= 16) return 1;
    if (variant.map_kind == KHM_MAP_SLICED_KV) return no("sliced-KV blocks hold at most 16 Q heads");
    if (coordinates <= 256) return 2;
    return no("gfx950 kernels hold at most 256 (token, head) coordinates per block");
}

}  // namespace khm

using namespace khm;

extern "C" int khm_sdpa_variant_sliced_kv(const khm_sdpa_config* config, uint32_t kv_tokens_per_iteration,
                                          uint32_t required_threads, uint32_t max_q_heads, khm_sdpa_variant* out) {
    clear_error();
    if (int status = validate_sdpa_config(config)) return status;
    KHM_REQUIRE(out != nullptr, "variant output must not be null");
    khm_sdpa_variant v{};
    v.map_kind = KHM_MAP_SLICED_KV;
    v.map_max_q_tokens = 1;
    v.map_max_q_heads = max_q_heads;
    v.map_kv_tokens_per_iteration = kv_tokens_per_iteration;
    v.map_required_threads = required_threads;
    v.kv_cache_tokens_per_page = config->tokens_per_page;
    sliced_kv_reduce_shape(*config, &v.reduce_max_q_tokens, &v.reduce_max_q_heads);
    v.reduce_required_threads = 256;
    KHM_REQUIRE(variant_supports(v, *config), "GQA SlicedKv execution variant does not support its config");
    *out = v;
    return KHM_OK;
}

extern "C" int khm_sdpa_variant_sliced_q(const khm_sdpa_config* config, uint32_t kind, uint32_t max_q_tokens,
                                         uint32_t kv_tokens_per_iteration, uint32_t max_q_heads, khm_sdpa_variant* out) {
    clear_error();
    if (int status = validate_sdpa_config(config)) return status;
    KHM_REQUIRE(out != nullptr, "variant output must not be null");
    KHM_REQUIRE(kind != KHM_MAP_SLICED_KV, "SlicedKv uses its own constructor");
    KHM_REQUIRE(max_q_tokens == 1 || max_q_tokens == 2 || max_q_tokens == 4 || max_q_tokens == 8 || max_q_tokens == 16 ||
                    max_q_tokens == 32,
                "GQA sliced-Q max_q_tokens must be one of 1, 2, 4, 8, 16, 32");
    KHM_REQUIRE(max_q_heads > 0 && max_q_heads <= q_heads_per_kv_head(*config),
                "GQA sliced-Q max_q_heads must be in 1..=q_heads_per_kv_head");
    uint64_t groups = 0;
    KHM_REQUIRE(sliced_q_simdgroups(kind, max_q_tokens, max_q_heads, &groups), "GQA tile geometry must fit u32");
    khm_sdpa_variant v{};
    v.map_kind = kind;
    v.map_max_q_tokens = max_q_tokens;
    v.map_max_q_heads = max_q_heads;
    v.map_kv_tokens_per_iteration = kv_tokens_per_iteration;
    v.map_required_threads = (uint32_t)(groups * 32);
    v.kv_cache_tokens_per_page = config->tokens_per_page;
    v.reduce_max_q_tokens = max_q_tokens;
    v.reduce_max_q_heads = 1;
    v.reduce_required_threads = v.map_required_threads;
    KHM_REQUIRE(variant_supports(v, *config), "GQA sliced-Q execution variant does not support its config");
    *out = v;
    return KHM_OK;
}

extern "C" int khm_sdpa_variant_supports(const khm_sdpa_variant* variant, const khm_sdpa_config* config) {
    clear_error();
    if (variant == nullptr || config == nullptr) return fail(KHM_ERR_INVALID_ARGUMENT, "variant and config must not be null");
    return variant_supports(*variant, *config) ? 1 : 0;
}

extern "C" int khm_sdpa_registry_new(const khm_sdpa_config* config, khm_sdpa_variant* variants, uint32_t capacity,
                                     uint32_t* count) {
    clear_error();
    if (int status = validate_sdpa_config(config)) return status;
    KHM_REQUIRE(count != nullptr, "registry count output must not be null");
    std::vector<khm_sdpa_variant> list;
    const uint32_t ratio = q_heads_per_kv_head(*config);
    {
        // sliced_kv_variant (sdpa.rs:311-319)
        uint32_t clamped = config->head_dim < 32 ? 32 : (config->head_dim > 256 ? 256 : config->head_dim);
        const uint32_t kv_tokens = next_power_of_two(clamped);
        khm_sdpa_variant v;
        if (int status = khm_sdpa_variant_sliced_kv(config, kv_tokens, kv_tokens < 128 ? kv_tokens : 128,
                                                    ratio < 8 ? ratio : 8, &v))
            return status;
        list.push_back(v);
    }
    const bool sliced_q = config->io_dtype == KHM_DTYPE_BF16 && sliced_q_profile(config->head_dim, config->tokens_per_page) &&
                          ratio <= 8;
    if (sliced_q) {
        const uint32_t cap = 256 / (8 / 8 * 32);  // max_sliced_q_heads(8)
        const uint32_t full = ratio < cap ? ratio : cap;
        auto per_head = [&](uint32_t tokens, uint32_t stage, uint32_t heads) -> int {
            khm_sdpa_variant v;
            if (int status = khm_sdpa_variant_sliced_q(config, KHM_MAP_Q_TOKENS_PER_HEAD, tokens, stage, heads, &v)) return status;
            list.push_back(v);
            return KHM_OK;
        };
        const bool d128 = config->head_dim == 128 && (config->tokens_per_page == 8 || config->tokens_per_page == 16);
        if (!d128) {
            const uint32_t half_ratio = div_ceil_u32(ratio, 2);
            const uint32_t half = half_ratio < cap ? half_ratio : cap;
            if (half != full) {
                if (int status = per_head(8, 16, half)) return status;
            }
        }
        if (int status = per_head(8, 16, full)) return status;
        if (config->head_dim == 256) {
            if (int status = per_head(8, 32, full)) return status;
        }
    }
    *count = (uint32_t)list.size();
    if (variants != nullptr) {
        if (capacity < list.size()) return fail(KHM_ERR_CAPACITY, "registry needs room for %zu variants", list.size());
        for (size_t i = 0; i < list.size(); ++i) variants[i] = list[i];
    }
    return KHM_OK;
}

extern "C" int khm_sdpa_variant_has_kernel(const khm_sdpa_config* config, const khm_sdpa_variant* variant, uint32_t kv_dtype) {
    clear_error();
    if (config == nullptr || variant == nullptr) return fail(KHM_ERR_INVALID_ARGUMENT, "variant and config must not be null");
    if (!variant_supports(*variant, *config)) {
        last_error_storage() = "variant does not support its config";
        return 0;
    }
    std::string why;
    const int family = kernel_family(*config, *variant, kv_dtype, &why);
    if (family == 0) last_error_storage() = why;
    return family != 0 ? 1 : 0;
}
