/*
 * CPU oracle for the paged GQA split-KV SDPA path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference's attention arithmetic.
 * It is the checker for the HIP kernels: only tests/, the smoke entry and the
 * cpu_baseline leg of bench.py may load it.  The product library never links,
 * loads or calls anything in this file.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout, crates/ prefix omitted where unambiguous):
 *
 *   khm_oracle_softmax            inference-executor-core/src/reference.rs:15-31
 *   khm_oracle_sigmoid            inference-executor-core/src/reference.rs:3-5
 *   khm_oracle_projected_gqa      inference-executor-core/src/attn/gqa/reference.rs:15-78
 *   khm_oracle_paged_gqa          same math, K/V gathered with the page formula of
 *                                 inference-backend-metal/src/components/metal/gqa_sdpa_sliced_kv_map.metal:13-19
 *                                 and the per-token visible window of
 *                                 .../metal/gqa_sdpa_sliced_q_map.metal:166-186
 *   khm_oracle_map_partials       partial-state semantics of gqa_sdpa_sliced_kv_map.metal:82-210
 *                                 and gqa_sdpa_sliced_q_map.metal:260-283 (normalized partial,
 *                                 natural-log max, canonical empty partial (0, -inf, 0))
 *   khm_oracle_reduce_sliced_kv   .../metal/gqa_sdpa_sliced_kv_reduce.metal:10-56
 *   khm_oracle_reduce_sliced_q    .../metal/gqa_sdpa_sliced_q_reduce.metal:4-63
 *   khm_oracle_gate_f32/_bf16     .../metal/gqa_activation_gate.metal:14-39
 *   khm_oracle_bf16_to_fp8_e4m3,
 *   khm_oracle_fp8_e4m3_to_bf16   inference-backend-metal/src/components/gqa/fp8.rs:19-58
 *   khm_oracle_f32_to_bf16        `half 2.7.1` bf16::from_f32 (round to nearest even, NaN kept quiet);
 *                                 call sites fp8.rs:11-17
 *
 * Parity pins (all exercised by tests/test_oracle.py): the closed-form causal case of
 * reference.rs:84-115, softmax [0, ln 3] -> [.25, .75] and sigmoid(0) = .5 of reference.rs:95-108,
 * the FP8 table / ties / exhaustive round trip / error bounds of fp8.rs:68-139, an independent
 * float64 numpy brute force on small shapes, torch scaled_dot_product_attention on medium
 * shapes, page-permutation invariance, and "any KV partition merges to the unsplit result".
 * No function in this file is "parity unpinned".
 *
 * Arithmetic is f32 in the reference's evaluation order (sequential dot products, softmax by
 * max-subtract / exp / sum / divide, value accumulation in token order).  Build with
 * -ffp-contract=off so no FMA contraction changes the rounding.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define KHM_ORACLE_KV_BF16 0u
#define KHM_ORACLE_KV_FP8_E4M3FN 1u

typedef struct khm_oracle_geom {
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint32_t tokens_per_page;
    uint32_t num_gqa_layers;
    uint32_t num_blocks;
    uint32_t num_page_ids_per_block;
    uint32_t kv_dtype; /* KHM_ORACLE_KV_* */
    uint64_t page_bytes;
    float scale;
    uint32_t reserved;
} khm_oracle_geom;

/* ---------------------------------------------------------------- scalar codecs */

static inline float bits_to_f32(uint32_t bits) {
    float value;
    memcpy(&value, &bits, sizeof value);
    return value;
}

static inline uint32_t f32_to_bits(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    return bits;
}

float khm_oracle_bf16_to_f32(uint16_t bits) { return bits_to_f32((uint32_t)bits << 16); }

uint16_t khm_oracle_f32_to_bf16(float value) {
    uint32_t bits = f32_to_bits(value);
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((bits >> 16) | 0x0040u); /* quiet NaN, payload truncated */
    }
    uint32_t rounding_bias = 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + rounding_bias) >> 16);
}

/* fp8.rs:19-45 */
uint8_t khm_oracle_bf16_to_fp8_e4m3(uint16_t bf16_bits) {
    float value = khm_oracle_bf16_to_f32(bf16_bits);
    uint8_t sign = (bf16_bits & 0x8000u) ? 0x80 : 0;
    float magnitude = fabsf(value);
    if (isnan(magnitude)) return sign | 0x7f;
    if (!isfinite(magnitude) || magnitude >= 448.0f) return sign | 0x7e;
    if (magnitude < 0x1p-6f) {
        uint8_t mantissa = (uint8_t)rintf(magnitude * 512.0f); /* rintf = ties-to-even in the default mode */
        return sign | (mantissa < 8 ? mantissa : 8);
    }
    int exponent = (int)floorf(log2f(magnitude));
    uint8_t mantissa = (uint8_t)rintf((magnitude * ldexpf(1.0f, -exponent) - 1.0f) * 8.0f);
    if (mantissa == 8) {
        exponent += 1;
        mantissa = 0;
    }
    int encoded_exponent = exponent + 7;
    if (encoded_exponent > 15 || (encoded_exponent == 15 && mantissa >= 7)) return sign | 0x7e;
    return sign | (uint8_t)(encoded_exponent << 3) | mantissa;
}

/* fp8.rs:47-58 */
uint16_t khm_oracle_fp8_e4m3_to_bf16(uint8_t bits) {
    uint32_t exponent = (bits >> 3) & 0x0f;
    uint32_t mantissa = bits & 0x07;
    if (exponent == 15 && mantissa == 7) {
        return (bits & 0x80) ? 0xffc0 : 0x7fc0;
    }
    float magnitude = exponent == 0 ? (float)mantissa / 512.0f
                                    : (1.0f + (float)mantissa / 8.0f) * ldexpf(1.0f, (int)exponent - 7);
    return khm_oracle_f32_to_bf16((bits & 0x80) ? -magnitude : magnitude);
}

/* reference.rs:3-5 */
float khm_oracle_sigmoid(float value) { return 1.0f / (1.0f + expf(-value)); }

/* reference.rs:15-31.  Returns 0 on success, -1 when the total is not finite and positive. */
int khm_oracle_softmax(const float* logits, uint64_t count, float* probabilities) {
    if (count == 0) return -1;
    float max_logit = -INFINITY;
    for (uint64_t i = 0; i < count; ++i) max_logit = logits[i] > max_logit ? logits[i] : max_logit;
    float total = 0.0f;
    for (uint64_t i = 0; i < count; ++i) {
        probabilities[i] = expf(logits[i] - max_logit);
        total += probabilities[i];
    }
    if (!(total > 0.0f) || !isfinite(total)) return -1;
    for (uint64_t i = 0; i < count; ++i) probabilities[i] = probabilities[i] / total;
    return 0;
}

/* ---------------------------------------------------------------- dense attention */

/*
 * One (query row, contiguous K/V window) attention: reference.rs:45-72.
 * k and v are [count][kv_stride] with the head's D values starting at k/v itself.
 * logits is scratch of `count` floats.  Value accumulation runs token-outer / dim-inner,
 * which visits every output dimension's terms in the same token order as the reference's
 * dim-outer loop, so each sum is bit-identical.
 */
static int attend_row(const float* q, const float* k, const float* v, uint64_t count, uint64_t kv_stride,
                      uint32_t head_dim, float scale, float* logits, float* out) {
    for (uint64_t t = 0; t < count; ++t) {
        const float* key = k + t * kv_stride;
        float dot_product = 0.0f;
        for (uint32_t d = 0; d < head_dim; ++d) dot_product += q[d] * key[d];
        logits[t] = dot_product * scale;
    }
    if (khm_oracle_softmax(logits, count, logits) != 0) return -1;
    for (uint32_t d = 0; d < head_dim; ++d) out[d] = 0.0f;
    for (uint64_t t = 0; t < count; ++t) {
        const float* value = v + t * kv_stride;
        const float probability = logits[t];
        for (uint32_t d = 0; d < head_dim; ++d) out[d] += probability * value[d];
    }
    return 0;
}

/*
 * reference.rs:15-78 (projected_gqa_reference).  q: [T][Hq][D]; k_by_req[r], v_by_req[r]:
 * [token_indices[r] + num_req_tokens][Hkv][D]; out: [T][Hq][D].
 */
int khm_oracle_projected_gqa(uint32_t num_reqs, const uint32_t* cu_tokens, const uint32_t* token_indices,
                             const float* q, const float* const* k_by_req, const float* const* v_by_req,
                             uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim, float scale,
                             float* out) {
    if (num_kv_heads == 0 || num_q_heads % num_kv_heads != 0 || cu_tokens[0] != 0) return -1;
    const uint32_t heads_per_kv_head = num_q_heads / num_kv_heads;
    const uint64_t kv_stride = (uint64_t)num_kv_heads * head_dim;
    int status = 0;
    for (uint32_t r = 0; r < num_reqs; ++r) {
        if (cu_tokens[r] > cu_tokens[r + 1]) return -1;
        const uint32_t req_start = cu_tokens[r];
        const uint32_t num_req_tokens = cu_tokens[r + 1] - req_start;
        const uint64_t context_length = (uint64_t)token_indices[r] + num_req_tokens;
        float* logits = (float*)malloc(sizeof(float) * (context_length ? context_length : 1));
        if (!logits) return -2;
        for (uint32_t i = 0; i < num_req_tokens; ++i) {
            const uint64_t token = req_start + i;
            const uint64_t visible = (uint64_t)token_indices[r] + i + 1;
            for (uint32_t h = 0; h < num_q_heads; ++h) {
                const uint32_t kv_head = h / heads_per_kv_head;
                const float* query = q + (token * num_q_heads + h) * head_dim;
                float* result = out + (token * num_q_heads + h) * head_dim;
                if (attend_row(query, k_by_req[r] + (uint64_t)kv_head * head_dim,
                               v_by_req[r] + (uint64_t)kv_head * head_dim, visible, kv_stride, head_dim, scale,
                               logits, result) != 0) {
                    status = -1;
                }
            }
        }
        free(logits);
    }
    return status;
}

/* ---------------------------------------------------------------- paged gather */

/* gqa_sdpa_sliced_kv_map.metal:13-19: byte offset of element (plane, kv_head, token, dim 0). */
static inline uint64_t page_element_offset(const khm_oracle_geom* g, const uint32_t* page_ids, uint32_t req_slot,
                                           uint32_t layer, uint32_t kv_head, uint64_t token, uint32_t plane) {
    const uint32_t tpp = g->tokens_per_page;
    const uint64_t block = token / ((uint64_t)tpp * g->num_page_ids_per_block);
    const uint64_t page_index = token / tpp % g->num_page_ids_per_block;
    const uint64_t table_index =
        ((((uint64_t)req_slot * g->num_gqa_layers + layer) * g->num_blocks + block) * g->num_page_ids_per_block)
        + page_index;
    const uint64_t page = page_ids[table_index];
    const uint64_t element_bytes = g->kv_dtype == KHM_ORACLE_KV_FP8_E4M3FN ? 1 : 2;
    return page * g->page_bytes
           + (((uint64_t)plane * g->num_kv_heads + kv_head) * tpp + token % tpp) * g->head_dim * element_bytes;
}

static void gather_rows(const khm_oracle_geom* g, const uint8_t* kv_pages, const uint32_t* page_ids,
                        uint32_t req_slot, uint32_t layer, uint32_t kv_head, uint64_t begin, uint64_t end,
                        uint32_t plane, float* rows) {
    for (uint64_t token = begin; token < end; ++token) {
        const uint8_t* source = kv_pages + page_element_offset(g, page_ids, req_slot, layer, kv_head, token, plane);
        float* row = rows + (token - begin) * g->head_dim;
        if (g->kv_dtype == KHM_ORACLE_KV_FP8_E4M3FN) {
            for (uint32_t d = 0; d < g->head_dim; ++d) {
                row[d] = khm_oracle_bf16_to_f32(khm_oracle_fp8_e4m3_to_bf16(source[d]));
            }
        } else {
            const uint16_t* values = (const uint16_t*)source;
            for (uint32_t d = 0; d < g->head_dim; ++d) row[d] = khm_oracle_bf16_to_f32(values[d]);
        }
    }
}

/*
 * Paged attention with a per-token visible window.  For flat Q token i the keys are the request-local
 * tokens [visible[2i], visible[2i+1]) of request slot req_slots[i], gathered through the page table,
 * then fed to the dense row routine above exactly as the reference tests build their expectation
 * (sliced_q_test.rs:179-205: an empty window yields zeros).
 * q: bf16 bits [T][Hq][D]; out: f32 [T][Hq][D].  num_threads <= 1 runs single-threaded.
 */
int khm_oracle_paged_gqa(const khm_oracle_geom* g, uint32_t num_tokens, const uint16_t* q, const uint8_t* kv_pages,
                         const uint32_t* req_slots, const uint32_t* page_ids, uint32_t layer,
                         const uint32_t* visible_ranges, float* out, int num_threads) {
    if (g->num_kv_heads == 0 || g->num_q_heads % g->num_kv_heads != 0) return -1;
    const uint32_t heads_per_kv_head = g->num_q_heads / g->num_kv_heads;
    const uint32_t D = g->head_dim;
    const int64_t num_units = (int64_t)num_tokens * g->num_kv_heads;
    int status = 0;
    (void)num_threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(num_threads > 1 ? num_threads : 1)
#endif
    for (int64_t unit = 0; unit < num_units; ++unit) {
        const uint32_t token = (uint32_t)(unit / g->num_kv_heads);
        const uint32_t kv_head = (uint32_t)(unit % g->num_kv_heads);
        const uint64_t begin = visible_ranges[2 * (uint64_t)token];
        const uint64_t end = visible_ranges[2 * (uint64_t)token + 1];
        float* result = out + ((uint64_t)token * g->num_q_heads + (uint64_t)kv_head * heads_per_kv_head) * D;
        if (end <= begin) {
            memset(result, 0, sizeof(float) * heads_per_kv_head * D);
            continue;
        }
        const uint64_t count = end - begin;
        float* k_rows = (float*)malloc(sizeof(float) * count * D);
        float* v_rows = (float*)malloc(sizeof(float) * count * D);
        float* logits = (float*)malloc(sizeof(float) * count);
        float* query = (float*)malloc(sizeof(float) * D);
        if (!k_rows || !v_rows || !logits || !query) {
            status = -2;
        } else {
            gather_rows(g, kv_pages, page_ids, req_slots[token], layer, kv_head, begin, end, 0, k_rows);
            gather_rows(g, kv_pages, page_ids, req_slots[token], layer, kv_head, begin, end, 1, v_rows);
            for (uint32_t j = 0; j < heads_per_kv_head; ++j) {
                const uint32_t h = kv_head * heads_per_kv_head + j;
                const uint16_t* q_bits = q + ((uint64_t)token * g->num_q_heads + h) * D;
                for (uint32_t d = 0; d < D; ++d) query[d] = khm_oracle_bf16_to_f32(q_bits[d]);
                if (attend_row(query, k_rows, v_rows, count, D, D, g->scale, logits, result + (uint64_t)j * D) != 0) {
                    status = -1;
                }
            }
        }
        free(k_rows);
        free(v_rows);
        free(logits);
        free(query);
    }
    return status;
}

/* ---------------------------------------------------------------- split-KV partial states */

/*
 * Partial state of one (map task template, flat Q token, Q head): softmax over the keys in
 * [max(kv_begin, visible_begin), min(kv_end, visible_end)).  Follows the Map kernels' contract:
 *   exp_sum   = sum_t exp(logit_t - max)           (0 when the intersection is empty)
 *   max_logit = natural-log running max            (-inf when exp_sum == 0)
 *   partial   = sum_t exp(logit_t - max) v_t / exp_sum   (0 when exp_sum == 0)
 * (gqa_sdpa_sliced_kv_map.metal:118-139,165,204; gqa_sdpa_sliced_q_map.metal:195-216,269-280).
 *
 * templates: [M][3] = (q_token_range_index, kv_begin, kv_end); q_token_ranges: [R][2] flat token
 * begin/end (for the sliced-KV kind pass ranges (i, i+1)).  Partial layout matches the kernels:
 * stats [M][Hq][max_q_tokens], partial [M][Hq][max_q_tokens][D] (max_q_tokens = 1 for sliced-KV).
 * Sentinel templates (range index >= num_ranges, e.g. u32::MAX) are skipped and leave memory untouched.
 * round_partials_bf16 != 0 rounds the normalized partial to bf16 as the reference's bf16 build does.
 */
int khm_oracle_map_partials(const khm_oracle_geom* g, uint32_t num_templates, const uint32_t* templates,
                            uint32_t num_ranges, const uint32_t* q_token_ranges, uint32_t max_q_tokens,
                            const uint16_t* q, const uint8_t* kv_pages, const uint32_t* req_slots,
                            const uint32_t* page_ids, uint32_t layer, const uint32_t* visible_ranges,
                            int round_partials_bf16, float* exp_sums, float* max_logits, float* partial) {
    const uint32_t heads_per_kv_head = g->num_q_heads / g->num_kv_heads;
    const uint32_t D = g->head_dim;
    for (uint32_t m = 0; m < num_templates; ++m) {
        const uint32_t range_index = templates[3 * (uint64_t)m];
        if (range_index >= num_ranges) continue;
        const uint32_t kv_begin = templates[3 * (uint64_t)m + 1];
        const uint32_t kv_end = templates[3 * (uint64_t)m + 2];
        const uint32_t flat_begin = q_token_ranges[2 * (uint64_t)range_index];
        const uint32_t flat_end = q_token_ranges[2 * (uint64_t)range_index + 1];
        for (uint32_t token = flat_begin; token < flat_end; ++token) {
            const uint32_t local_token = token - flat_begin;
            if (local_token >= max_q_tokens) return -1;
            uint64_t begin = visible_ranges[2 * (uint64_t)token];
            uint64_t end = visible_ranges[2 * (uint64_t)token + 1];
            if (begin < kv_begin) begin = kv_begin;
            if (end > kv_end) end = kv_end;
            const uint64_t count = end > begin ? end - begin : 0;
            float* k_rows = (float*)malloc(sizeof(float) * (count ? count : 1) * D);
            float* v_rows = (float*)malloc(sizeof(float) * (count ? count : 1) * D);
            float* logits = (float*)malloc(sizeof(float) * (count ? count : 1));
            if (!k_rows || !v_rows || !logits) return -2;
            for (uint32_t h = 0; h < g->num_q_heads; ++h) {
                const uint32_t kv_head = h / heads_per_kv_head;
                const uint64_t state = ((uint64_t)m * g->num_q_heads + h) * max_q_tokens + local_token;
                float* numerator = partial + state * D;
                for (uint32_t d = 0; d < D; ++d) numerator[d] = 0.0f;
                if (count == 0) {
                    exp_sums[state] = 0.0f;
                    max_logits[state] = -INFINITY;
                    continue;
                }
                if (h % heads_per_kv_head == 0) {
                    gather_rows(g, kv_pages, page_ids, req_slots[token], layer, kv_head, begin, end, 0, k_rows);
                    gather_rows(g, kv_pages, page_ids, req_slots[token], layer, kv_head, begin, end, 1, v_rows);
                }
                const uint16_t* q_bits = q + ((uint64_t)token * g->num_q_heads + h) * D;
                float max_logit = -INFINITY;
                for (uint64_t t = 0; t < count; ++t) {
                    float dot_product = 0.0f;
                    for (uint32_t d = 0; d < D; ++d) dot_product += khm_oracle_bf16_to_f32(q_bits[d]) * k_rows[t * D + d];
                    logits[t] = dot_product * g->scale;
                    max_logit = logits[t] > max_logit ? logits[t] : max_logit;
                }
                float exp_sum = 0.0f;
                for (uint64_t t = 0; t < count; ++t) {
                    const float weight = expf(logits[t] - max_logit);
                    exp_sum += weight;
                    for (uint32_t d = 0; d < D; ++d) numerator[d] += weight * v_rows[t * D + d];
                }
                exp_sums[state] = exp_sum;
                max_logits[state] = exp_sum > 0.0f ? max_logit : -INFINITY;
                for (uint32_t d = 0; d < D; ++d) {
                    float value = exp_sum > 0.0f ? numerator[d] / exp_sum : 0.0f;
                    if (round_partials_bf16) value = khm_oracle_bf16_to_f32(khm_oracle_f32_to_bf16(value));
                    numerator[d] = value;
                }
            }
            free(k_rows);
            free(v_rows);
            free(logits);
        }
    }
    return 0;
}

/*
 * gqa_sdpa_sliced_kv_reduce.metal:10-56.  stats [M][Hq]; partial [M][Hq][D]; cu [T+1]; out [T][Hq][D].
 */
void khm_oracle_reduce_sliced_kv(const float* exp_sums, const float* max_logits, const float* partial,
                                 const uint32_t* cu_partial_outputs, uint32_t num_tokens, uint32_t num_q_heads,
                                 uint32_t head_dim, float* out) {
    for (uint32_t token = 0; token < num_tokens; ++token) {
        const uint32_t begin = cu_partial_outputs[token];
        const uint32_t end = cu_partial_outputs[token + 1];
        for (uint32_t h = 0; h < num_q_heads; ++h) {
            float global_max = -INFINITY;
            for (uint32_t p = begin; p < end; ++p) {
                const float value = max_logits[(uint64_t)p * num_q_heads + h];
                global_max = value > global_max ? value : global_max;
            }
            for (uint32_t d = 0; d < head_dim; ++d) {
                float global_exp_sum = 0.0f;
                float accumulator = 0.0f;
                for (uint32_t p = begin; p < end; ++p) {
                    const uint64_t state = (uint64_t)p * num_q_heads + h;
                    const float weight = isfinite(max_logits[state]) ? expf(max_logits[state] - global_max) * exp_sums[state] : 0.0f;
                    global_exp_sum += weight;
                    accumulator += weight * partial[state * head_dim + d];
                }
                out[((uint64_t)token * num_q_heads + h) * head_dim + d] =
                    global_exp_sum > 0.0f ? accumulator / global_exp_sum : 0.0f;
            }
        }
    }
}

/*
 * gqa_sdpa_sliced_q_reduce.metal:4-63.  stats [M][Hq][max_q_tokens]; partial [M][Hq][max_q_tokens][D];
 * q_token_ranges [R][2]; cu [R+1]; out [T][Hq][D] (only tokens covered by the ranges are written).
 */
void khm_oracle_reduce_sliced_q(const float* exp_sums, const float* max_logits, const float* partial,
                                const uint32_t* q_token_ranges, const uint32_t* cu_partial_outputs,
                                uint32_t num_ranges, uint32_t max_q_tokens, uint32_t num_q_heads, uint32_t head_dim,
                                float* out) {
    for (uint32_t r = 0; r < num_ranges; ++r) {
        const uint32_t flat_begin = q_token_ranges[2 * (uint64_t)r];
        const uint32_t flat_end = q_token_ranges[2 * (uint64_t)r + 1];
        const uint32_t begin = cu_partial_outputs[r];
        const uint32_t end = cu_partial_outputs[r + 1];
        for (uint32_t h = 0; h < num_q_heads; ++h) {
            for (uint32_t local = 0; local < flat_end - flat_begin; ++local) {
                float global_max = -INFINITY;
                for (uint32_t p = begin; p < end; ++p) {
                    const float value = max_logits[((uint64_t)p * num_q_heads + h) * max_q_tokens + local];
                    global_max = value > global_max ? value : global_max;
                }
                for (uint32_t d = 0; d < head_dim; ++d) {
                    float global_sum = 0.0f;
                    float accumulator = 0.0f;
                    for (uint32_t p = begin; p < end; ++p) {
                        const uint64_t state = ((uint64_t)p * num_q_heads + h) * max_q_tokens + local;
                        const float weight = exp_sums[state] == 0.0f ? 0.0f : expf(max_logits[state] - global_max) * exp_sums[state];
                        global_sum += weight;
                        accumulator += weight * partial[state * head_dim + d];
                    }
                    out[((uint64_t)(flat_begin + local) * num_q_heads + h) * head_dim + d] =
                        global_sum > 0.0f ? accumulator / global_sum : 0.0f;
                }
            }
        }
    }
}

/* ---------------------------------------------------------------- sigmoid gate */

/* gqa_activation_gate.metal:14-17,28-39 (f32 build). */
void khm_oracle_gate_f32(const float* attention, const float* gates, uint64_t count, float* out) {
    for (uint64_t i = 0; i < count; ++i) {
        const float x = gates[i];
        const float y = 1.0f / (1.0f + expf(-fabsf(x)));
        out[i] = attention[i] * (x < 0.0f ? 1.0f - y : y);
    }
}

static inline float round_bf16(float value) { return khm_oracle_bf16_to_f32(khm_oracle_f32_to_bf16(value)); }

/* gqa_activation_gate.metal:6-12,19-26,28-39 (bf16 build): every intermediate is rounded to bf16. */
void khm_oracle_gate_bf16(const uint16_t* attention, const uint16_t* gates, uint64_t count, uint16_t* out) {
    for (uint64_t i = 0; i < count; ++i) {
        const float x = khm_oracle_bf16_to_f32(gates[i]);
        const float abs_x = round_bf16(fabsf(x));
        const float neg_abs_x = round_bf16(-abs_x);
        const float exp_x = round_bf16(expf(neg_abs_x));
        const float denom = round_bf16(1.0f + exp_x);
        const float y = round_bf16(1.0f / denom);
        const float sigmoid = x < 0.0f ? round_bf16(1.0f - y) : y;
        out[i] = khm_oracle_f32_to_bf16(khm_oracle_bf16_to_f32(attention[i]) * sigmoid);
    }
}

int khm_oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
