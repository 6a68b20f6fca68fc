/*
 * C ABI of the MI355X (gfx950) paged GQA split-KV SDPA backend component.
 *
 * This header is the drop-in boundary: plain C types, raw device pointers and byte
 * lengths, no framework types.  Every entry point names the reference interface it
 * replaces (paths relative to the reference checkout).  Kernel launches are enqueued
 * on the caller's hipStream_t (passed as void*) and never synchronize, matching the
 * reference rule that an Operator records work and never submits
 * (docs/executor_gqa.md:423-424).
 *
 * Error model: the reference panics on internal invariants (docs/high_level.md:36-47).
 * Here every function returns a khm_status (0 = ok, negative = error) and
 * khm_last_error() returns the message, which repeats the reference's assertion text
 * where one exists, so a binding can re-raise it as a panic.
 *
 * Threading: handles are not thread-safe (the reference uses Rc/RefCell and a
 * thread-local pipeline cache: crates/inference-backend-metal/src/metal/kernel.rs:26-30).
 */
#ifndef KHM_GQA_SDPA_H
#define KHM_GQA_SDPA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum khm_status {
    KHM_OK = 0,
    KHM_ERR_INVALID_ARGUMENT = -1, /* a reference assert!/panic! condition */
    KHM_ERR_UNSUPPORTED = -2,      /* legal in the reference, not built for gfx950 (see khm_last_error) */
    KHM_ERR_HIP = -3,              /* a HIP runtime call failed */
    KHM_ERR_CAPACITY = -4          /* caller-provided output array too small */
} khm_status;

/* Message of the last failing call on this thread ("" when none). */
const char* khm_last_error(void);
/* Library version string. */
const char* khm_version(void);

/* crates/inference-backend-metal/src/metal Dtype, restricted to what this path moves. */
typedef enum khm_dtype {
    KHM_DTYPE_F32 = 0,
    KHM_DTYPE_BF16 = 1,
    KHM_DTYPE_FP8_E4M3FN = 2,
    KHM_DTYPE_U32 = 3
} khm_dtype;

/* ReplayU32::{Fixed, Parameter} (crates/inference-backend-metal/src/metal/stream/parameter.rs:27-47).
 * A Parameter is an index into a device-resident u32 parameter block that the caller rewrites
 * before each submission; kernels read it at run time, so one recorded launch sequence (or a
 * captured hipGraph) serves every active count. */
typedef struct khm_replay_u32 {
    uint32_t is_parameter; /* 0 = Fixed(value), 1 = Parameter(value = index into the block) */
    uint32_t value;
} khm_replay_u32;

/* Borrowed device buffer: base pointer + length, validated against the minimum the launch needs
 * (the reference asserts Buffer::len_bytes in Invocation::validate, sliced_kv.rs:594-613). */
typedef struct khm_buffer {
    void* ptr;
    uint64_t len_bytes;
} khm_buffer;

/* PageTableLayout (components/gqa/kv_page_write.rs:34-58) ==
 * GQAPageTableLayout (crates/inference-executor-metal/src/attn/gqa/request_page_table.rs:7-44).
 * page_ids is a u32 tensor [num_req_slots][num_gqa_layers][num_blocks][num_page_ids_per_block]. */
typedef struct khm_page_table_layout {
    uint32_t num_req_slots;
    uint32_t num_gqa_layers;
    uint32_t num_blocks;
    uint32_t num_page_ids_per_block;
} khm_page_table_layout;

/* ------------------------------------------------------------------------------------------
 * Static capability: components/gqa/sdpa.rs
 * ------------------------------------------------------------------------------------------ */

/* sdpa::MapKernelKind (sdpa.rs:22-28). */
typedef enum khm_map_kernel_kind {
    KHM_MAP_SLICED_KV = 0,
    KHM_MAP_Q_TOKENS_PER_HEAD = 1,
    KHM_MAP_Q_HEADS_PER_TOKEN = 2,
    KHM_MAP_Q_TOKENS_AND_HEADS = 3
} khm_map_kernel_kind;

/* sdpa::Config (sdpa.rs:219-227). */
typedef struct khm_sdpa_config {
    uint32_t io_dtype; /* khm_dtype: F32 or BF16 */
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint32_t tokens_per_page;
} khm_sdpa_config;

/* sdpa::ExecutionVariant = MapKernelConstants + ReduceKernelConstants (sdpa.rs:6-57), flattened.
 * required_threads keeps the reference's meaning (32 lanes per SIMDgroup); the gfx950 launch
 * width is derived by the backend and is not part of the ABI. */
typedef struct khm_sdpa_variant {
    uint32_t map_kind; /* khm_map_kernel_kind */
    uint32_t map_max_q_tokens;
    uint32_t map_max_q_heads;
    uint32_t map_kv_tokens_per_iteration;
    uint32_t map_required_threads;
    uint32_t kv_cache_tokens_per_page;
    uint32_t reduce_max_q_tokens;
    uint32_t reduce_max_q_heads;
    uint32_t reduce_required_threads;
} khm_sdpa_variant;

/* ExecutionVariant::sliced_kv (sdpa.rs:60-90). */
int khm_sdpa_variant_sliced_kv(const khm_sdpa_config* config, uint32_t kv_tokens_per_iteration,
                               uint32_t required_threads, uint32_t max_q_heads, khm_sdpa_variant* out);
/* ExecutionVariant::sliced_q / sliced_q_per_head (sdpa.rs:92-160). */
int khm_sdpa_variant_sliced_q(const khm_sdpa_config* config, uint32_t kind, uint32_t max_q_tokens,
                              uint32_t kv_tokens_per_iteration, uint32_t max_q_heads, khm_sdpa_variant* out);
/* ExecutionVariant::supports (sdpa.rs:162-215): 1 = supported, 0 = not, negative = error. */
int khm_sdpa_variant_supports(const khm_sdpa_variant* variant, const khm_sdpa_config* config);
/* Registry::new (sdpa.rs:248-267): writes the default legal variants; *count receives how many. */
int khm_sdpa_registry_new(const khm_sdpa_config* config, khm_sdpa_variant* variants, uint32_t capacity,
                          uint32_t* count);
/* 1 when this build has a gfx950 kernel for (config, variant, kv_dtype), else 0 with the reason in
 * khm_last_error().  The reference has no counterpart: its kernels are JIT-specialised for any geometry. */
int khm_sdpa_variant_has_kernel(const khm_sdpa_config* config, const khm_sdpa_variant* variant, uint32_t kv_dtype);

/* ------------------------------------------------------------------------------------------
 * Component configuration shared by sliced_kv::Config (sdpa/sliced_kv.rs:91-99) and
 * sliced_q::Config (sdpa/sliced_q.rs:171-179).  The reference hard-wires FP8 E4M3FN K/V pages
 * and io-dtype partials; kv_dtype and partial_dtype make both explicit:
 *   kv_dtype      BF16 (16-bit pages) or FP8_E4M3FN (the reference's 8-bit pages)
 *   partial_dtype BF16 (the reference's scratch layout, gqa_sdpa_sliced_kv_map.metal:204) or
 *                 F32 (allowed when this backend owns the scratch)
 * num_tokens_per_page = page_bytes / (2 * num_kv_heads * head_dim * sizeof(kv element))
 * (sliced_kv.rs:113-125 with the element size generalised).
 * ------------------------------------------------------------------------------------------ */
typedef struct khm_gqa_sdpa_config {
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    float scale;
    uint32_t page_bytes;
    khm_page_table_layout page_table_layout;
    uint32_t dtype;         /* io dtype of q / output: KHM_DTYPE_BF16 */
    uint32_t kv_dtype;      /* KHM_DTYPE_BF16 or KHM_DTYPE_FP8_E4M3FN */
    uint32_t partial_dtype; /* KHM_DTYPE_BF16 or KHM_DTYPE_F32 */
} khm_gqa_sdpa_config;

/* sliced_kv::Shape (sliced_kv.rs:215-219) and sliced_q::Shape (sliced_q.rs:248-253).
 * num_total_q_token_tiles is ignored by the sliced-KV component. */
typedef struct khm_gqa_sdpa_shape {
    uint32_t num_total_tokens;
    uint32_t num_total_q_token_tiles;
    uint32_t num_total_sdpa_map_task_templates;
} khm_gqa_sdpa_shape;

/* Config::num_tokens_per_page; 0 on invalid config. */
uint32_t khm_gqa_sdpa_num_tokens_per_page(const khm_gqa_sdpa_config* config);
/* Config::q_bytes (sliced_kv.rs:168-172, sliced_q.rs:214-224). */
uint64_t khm_gqa_sdpa_q_bytes(const khm_gqa_sdpa_config* config, const khm_gqa_sdpa_shape* shape);
/* Config::page_ids_bytes (sliced_kv.rs:184-186). */
uint64_t khm_gqa_sdpa_page_ids_bytes(const khm_gqa_sdpa_config* config);

/* ------------------------------------------------------------------------------------------
 * Sliced-KV component: sdpa/sliced_kv.rs (decode-style split-KV Map + flat Reduce)
 * ------------------------------------------------------------------------------------------ */
typedef struct khm_sliced_kv khm_sliced_kv; /* sliced_kv::Compute */

/* MapBuffers (sliced_kv.rs:237-247); kernel bindings 0..7 of gqa_sdpa_sliced_kv_map.metal:36-45. */
typedef struct khm_sliced_kv_map_buffers {
    khm_buffer q;                       /* io dtype [T][Hq][D] */
    khm_buffer kv_pages;                /* bytes [P][page_bytes], page = [K|V][Hkv][tokens_per_page][D] */
    khm_buffer req_slots;               /* u32 [T] */
    khm_buffer page_ids;                /* u32 page table */
    khm_buffer sdpa_map_task_templates; /* u32 [M][3] = (q_token, kv_begin, kv_end); u32::MAX padded */
    khm_buffer partial_exp_sums;        /* f32 [M][Hq] */
    khm_buffer partial_max_logits;      /* f32 [M][Hq], natural log */
    khm_buffer partial_output;          /* partial_dtype [M][Hq][D], normalized */
} khm_sliced_kv_map_buffers;

/* ReduceBuffers (sliced_kv.rs:249-256). */
typedef struct khm_sliced_kv_reduce_buffers {
    khm_buffer partial_exp_sums;
    khm_buffer partial_max_logits;
    khm_buffer partial_output;
    khm_buffer cu_sdpa_partial_outputs; /* u32 [T+1] */
    khm_buffer output;                  /* io dtype [T][Hq][D] */
} khm_sliced_kv_reduce_buffers;

/* Config::partial_output_stats_bytes / partial_output_bytes (sliced_kv.rs:202-212). */
uint64_t khm_sliced_kv_partial_output_stats_bytes(const khm_gqa_sdpa_config* config, const khm_gqa_sdpa_shape* shape);
uint64_t khm_sliced_kv_partial_output_bytes(const khm_gqa_sdpa_config* config, const khm_gqa_sdpa_shape* shape);

/* Compute::new (sliced_kv.rs:322-355): validates config/variant/shape and selects the ahead-of-time
 * compiled kernel for the geometry (kernel identity does not depend on the shape, as the reference
 * tests in sliced_kv_test.rs:20-42). */
int khm_sliced_kv_create(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                         const khm_gqa_sdpa_shape* shape, khm_sliced_kv** out);
void khm_sliced_kv_destroy(khm_sliced_kv* compute);
/* Opaque identity of the selected Map / Reduce kernels (for the pipeline-reuse test). */
const void* khm_sliced_kv_map_kernel_id(const khm_sliced_kv* compute);
const void* khm_sliced_kv_reduce_kernel_id(const khm_sliced_kv* compute);

/* Compute::invoke_map + MapInvocation::record (sliced_kv.rs:357-377,558-592): grid
 * (num_total_sdpa_map_task_templates, Hkv * q_head_ranges).  replay_parameters is the device u32
 * parameter block (may be NULL when every khm_replay_u32 is Fixed). */
int khm_sliced_kv_map(const khm_sliced_kv* compute, const khm_sliced_kv_map_buffers* buffers,
                      khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                      khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream);
/* Compute::invoke_reduce + ReduceInvocation::record (sliced_kv.rs:379-388,623-638). */
int khm_sliced_kv_reduce(const khm_sliced_kv* compute, const khm_sliced_kv_reduce_buffers* buffers,
                         khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream);
/* Reduce fused with the sigmoid gate that follows it in GQA::record
 * (crates/inference-executor-metal/src/attn/gqa/backend.rs:332-434): output = bf16(attn) * sigmoid(gate)
 * with the bf16 step rounding of gqa_activation_gate.metal:19-39.  gates: io dtype [T][Hq][D]. */
int khm_sliced_kv_reduce_gated(const khm_sliced_kv* compute, const khm_sliced_kv_reduce_buffers* buffers,
                               khm_buffer gates, khm_replay_u32 num_active_tokens,
                               const uint32_t* replay_parameters, void* stream);

/* Map and Reduce in one launch.  The reference records two operators with a barrier between them
 * (attn/gqa/backend.rs:458-482); on gfx950 the second launch and its dependent loads cost several
 * microseconds of a ~100 us decode step, so the last Map block to finish a (token, KV head) merges that
 * token's partial states itself.  Same partial buffers and merge formula as khm_sliced_kv_map followed by
 * khm_sliced_kv_reduce[_gated]; only the summation order of the merge differs.
 *   arrival_counters  u32 [num_total_tokens][Hkv * q_head_ranges], all zero before the first launch; every
 *                     launch leaves them zero again, so one memset at allocation is enough.  Launches that
 *                     share the counters must not overlap.
 *   gates             optional (ptr == NULL: no gate). */
uint64_t khm_sliced_kv_arrival_counters_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                              const khm_gqa_sdpa_shape* shape);
int khm_sliced_kv_map_reduce(const khm_sliced_kv* compute, const khm_sliced_kv_map_buffers* map_buffers,
                             const khm_sliced_kv_reduce_buffers* reduce_buffers, khm_buffer gates,
                             khm_buffer arrival_counters, khm_replay_u32 page_table_index,
                             khm_replay_u32 num_active_tokens, khm_replay_u32 num_active_kv_splits,
                             const uint32_t* replay_parameters, void* stream);

/* khm_sliced_kv_map_reduce for callers that cannot allocate or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its executor owns a Scratch,
 * sliced_kv.rs:265-320).  The partial states and the arrival counters live in a device array owned by the library,
 * khm_sliced_kv_static_scratch_bytes() = 16 MiB per GPU, held until the process ends; the call allocates and frees
 * nothing and enqueues two kernels on `stream` (a clear of the arrival counters, then the fused Map + Reduce).
 * A shape whose partial states (two f32 [M][Hq] statistics + partial_dtype [M][Hq][D], each rounded up to 256 bytes)
 * exceed 16 MiB - 256 KiB, or whose arrival counters (u32 [T][Hkv * q_head_ranges]) exceed 256 KiB, is rejected with
 * KHM_ERR_INVALID_ARGUMENT.  Every call on one GPU shares that GPU's array: calls that overlap in time on one GPU
 * race, whatever their streams; calls on one stream, or otherwise ordered, are fine.  Results are those of
 * khm_sliced_kv_map_reduce bit for bit. */
typedef struct khm_sliced_kv_static_buffers {
    khm_buffer q;                       /* io dtype [T][Hq][D] */
    khm_buffer kv_pages;
    khm_buffer req_slots;               /* u32 [T] */
    khm_buffer page_ids;
    khm_buffer sdpa_map_task_templates; /* u32 [M][3] */
    khm_buffer cu_sdpa_partial_outputs; /* u32 [T+1] */
    khm_buffer output;                  /* io dtype [T][Hq][D] */
} khm_sliced_kv_static_buffers;
uint64_t khm_sliced_kv_static_scratch_bytes(void);
int khm_sliced_kv_map_reduce_static(const khm_sliced_kv* compute, const khm_sliced_kv_static_buffers* buffers,
                                    khm_buffer gates, khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                    khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * Sliced-Q component: sdpa/sliced_q.rs (verify blocks and chunked prefill)
 * ------------------------------------------------------------------------------------------ */
typedef struct khm_sliced_q khm_sliced_q; /* sliced_q::Compute */

/* MapBuffers (sliced_q.rs:284-297); bindings of gqa_sdpa_sliced_q_map.metal:29-43. */
typedef struct khm_sliced_q_map_buffers {
    khm_buffer q;
    khm_buffer kv_pages;
    khm_buffer req_slots;
    khm_buffer page_ids;
    khm_buffer visible_kv_token_ranges; /* u32 [T][2], request-local half-open */
    khm_buffer q_token_ranges;          /* u32 [R][2], flat token begin/end */
    khm_buffer sdpa_map_task_templates; /* u32 [M][3] = (q_token_range, kv_begin, kv_end) */
    khm_buffer partial_output;          /* partial_dtype [M][Hq][max_q_tokens][D] */
    khm_buffer partial_exp_sums;        /* f32 [M][Hq][max_q_tokens] */
    khm_buffer partial_max_logits;
} khm_sliced_q_map_buffers;

/* DirectBuffers (sliced_q.rs:299-311). */
typedef struct khm_sliced_q_direct_buffers {
    khm_buffer q;
    khm_buffer kv_pages;
    khm_buffer req_slots;
    khm_buffer page_ids;
    khm_buffer visible_kv_token_ranges;
    khm_buffer q_token_ranges;
    khm_buffer sdpa_map_task_templates;
    khm_buffer output; /* io dtype [T][Hq][D] */
} khm_sliced_q_direct_buffers;

/* ReduceBuffers (sliced_q.rs:313-321). */
typedef struct khm_sliced_q_reduce_buffers {
    khm_buffer partial_output;
    khm_buffer partial_exp_sums;
    khm_buffer partial_max_logits;
    khm_buffer q_token_ranges;
    khm_buffer cu_sdpa_partial_outputs; /* u32 [R+1] */
    khm_buffer output;
} khm_sliced_q_reduce_buffers;

/* Config::partial_output_bytes / partial_output_stats_bytes (sliced_q.rs:226-232,78-101). */
uint64_t khm_sliced_q_partial_output_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                           const khm_gqa_sdpa_shape* shape);
uint64_t khm_sliced_q_partial_output_stats_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                                 const khm_gqa_sdpa_shape* shape);

/* Compute::new / Compute::new_direct (sliced_q.rs:356-415). */
int khm_sliced_q_create(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                        const khm_gqa_sdpa_shape* shape, int direct_output, khm_sliced_q** out);
void khm_sliced_q_destroy(khm_sliced_q* compute);
const void* khm_sliced_q_map_kernel_id(const khm_sliced_q* compute);

/* Compute::invoke_map + MapInvocation::record (sliced_q.rs:417-449,547-593). */
int khm_sliced_q_map(const khm_sliced_q* compute, const khm_sliced_q_map_buffers* buffers,
                     khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                     khm_replay_u32 num_active_q_token_tiles, khm_replay_u32 num_active_kv_splits,
                     const uint32_t* replay_parameters, void* stream);
/* Compute::invoke_direct (sliced_q.rs:451-482): one full-range template per Q range, final output. */
int khm_sliced_q_direct(const khm_sliced_q* compute, const khm_sliced_q_direct_buffers* buffers,
                        khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                        khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream);
/* Compute::invoke_reduce + ReduceInvocation::record (sliced_q.rs:484-504,620-642). */
int khm_sliced_q_reduce(const khm_sliced_q* compute, const khm_sliced_q_reduce_buffers* buffers,
                        khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream);
/* The same two calls fused with the sigmoid gate that follows the SDPA in GQA::record
 * (crates/inference-executor-metal/src/attn/gqa/backend.rs:413-421; activation_gate.rs:35-168,
 * gqa_activation_gate.metal:19-39): output = bf16(attn) * sigmoid(gate) with the kernel's bf16 step rounding, so the
 * result equals khm_sliced_q_direct / khm_sliced_q_reduce followed by khm_gqa_activation_gate bit for bit, without the
 * extra pass over the output.  gates: bf16 [T][Hq][D]. */
int khm_sliced_q_direct_gated(const khm_sliced_q* compute, const khm_sliced_q_direct_buffers* buffers, khm_buffer gates,
                              khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                              khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream);
int khm_sliced_q_reduce_gated(const khm_sliced_q* compute, const khm_sliced_q_reduce_buffers* buffers, khm_buffer gates,
                              khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream);

/* Map and Reduce in one launch for the sliced-Q component; see khm_sliced_kv_map_reduce.
 *   arrival_counters  u32 [num_total_q_token_tiles][Hkv * q_head_ranges], zero before the first launch. */
uint64_t khm_sliced_q_arrival_counters_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                             const khm_gqa_sdpa_shape* shape);
int khm_sliced_q_map_reduce(const khm_sliced_q* compute, const khm_sliced_q_map_buffers* map_buffers,
                            const khm_sliced_q_reduce_buffers* reduce_buffers, khm_buffer arrival_counters,
                            khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                            khm_replay_u32 num_active_q_token_tiles, khm_replay_u32 num_active_kv_splits,
                            const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * Sigmoid gate: components/gqa/activation_gate.rs:35-168, gqa_activation_gate.metal:14-59
 * out = attention * sigmoid(gate) over [num_active_tokens][Hq][D]; dtype F32 or BF16.
 * ------------------------------------------------------------------------------------------ */
int khm_gqa_activation_gate(uint32_t dtype, uint32_t num_q_heads, uint32_t head_dim, uint32_t num_total_tokens,
                            khm_buffer attention_output, khm_buffer gates, khm_buffer output,
                            khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * Split of the fused input projection, the first launch of the layer (attn/gqa/backend.rs:358-370):
 * components/gqa/qgkv_split.rs:34-236 with gqa_qgkv_split.metal:5-44 (a token's row is
 * [Hq x (q head | gate head)][Hkv x k head][Hkv x v head]) and components/gqa/qkv_split.rs with
 * gqa_qkv_split.metal:5-34 ([Hq x q head][Hkv x k head][Hkv x v head]).  The first num_active_tokens rows go to
 * q, g [T][Hq][D] and k, v [T][Hkv][D]; rows beyond stay untouched.  dtype F32 or BF16; bit-exact.
 * Buffers must be aligned to their element size; 16-byte alignment gives the widest copies.
 * ------------------------------------------------------------------------------------------ */
typedef struct khm_gqa_projection_split_config {
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint32_t dtype; /* KHM_DTYPE_F32 or KHM_DTYPE_BF16 */
} khm_gqa_projection_split_config;
/* Config::qgkv_width / qkv_width: elements of one token's projection row (0: the head count does not fit u32). */
uint64_t khm_gqa_qgkv_width(const khm_gqa_projection_split_config* config);
uint64_t khm_gqa_qkv_width(const khm_gqa_projection_split_config* config);
int khm_gqa_qgkv_split(const khm_gqa_projection_split_config* config, uint32_t num_total_tokens, khm_buffer qgkv,
                       khm_buffer q, khm_buffer g, khm_buffer k, khm_buffer v, khm_replay_u32 num_active_tokens,
                       const uint32_t* replay_parameters, void* stream);
int khm_gqa_qkv_split(const khm_gqa_projection_split_config* config, uint32_t num_total_tokens, khm_buffer qkv,
                      khm_buffer q, khm_buffer k, khm_buffer v, khm_replay_u32 num_active_tokens,
                      const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * FP8 E4M3FN unit-scale codec, host side: components/gqa/fp8.rs:19-58
 * ------------------------------------------------------------------------------------------ */
uint8_t khm_bf16_to_fp8_e4m3(uint16_t bf16_bits);
uint16_t khm_fp8_e4m3_to_bf16(uint8_t fp8_bits);
uint16_t khm_f32_to_bf16(float value);
float khm_bf16_to_f32(uint16_t bf16_bits);
/* The same codec on the device, element-wise over `count` values: decode is what the Map kernels apply to FP8 pages
 * (fp8_e4m3x8_to_bf16x8, components/metal/gqa_fp8.metal:1-25), encode is what the page writer applies
 * (bf16_to_fp8_e4m3, components/metal/gqa_kv_page_write.metal:5-31).  The 8-bit buffer (`codes`) must be 8-byte and the
 * 16-bit buffer (`bf16_out`, `bf16_in`) 16-byte aligned. */
int khm_fp8_e4m3_to_bf16_device(khm_buffer codes, khm_buffer bf16_out, uint64_t count, void* stream);
int khm_bf16_to_fp8_e4m3_device(khm_buffer bf16_in, khm_buffer codes, uint64_t count, void* stream);

/* ------------------------------------------------------------------------------------------
 * K/V page writer: components/gqa/kv_page_write.rs:60-283, gqa_kv_page_write.metal:33-110
 * Scatters the bf16 K and V rows [W][Hkv][D] of W token writes through the page table into pages laid out
 * [K|V][Hkv][tokens_per_page][D].  The reference writes FP8 E4M3FN pages only; kv_dtype BF16 writes 16-bit pages.
 * ------------------------------------------------------------------------------------------ */
/* kv_page_write::Config (kv_page_write.rs:60-66) plus the page element type. */
typedef struct khm_kv_page_write_config {
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint32_t page_bytes;
    uint32_t dtype;    /* source tensors: KHM_DTYPE_BF16 */
    uint32_t kv_dtype; /* pages: KHM_DTYPE_FP8_E4M3FN (reference) or KHM_DTYPE_BF16 */
} khm_kv_page_write_config;
/* kv_page_write::Shape (kv_page_write.rs:115-119). */
typedef struct khm_kv_page_write_shape {
    uint32_t num_total_token_writes;
    khm_page_table_layout page_table_layout;
} khm_kv_page_write_shape;
/* kv_page_write::Buffers (kv_page_write.rs:136-145): flat_k/flat_v bf16 [W][Hkv][D], req_slots/flat_token_indices u32 [W]. */
typedef struct khm_kv_page_write_buffers {
    khm_buffer pages;
    khm_buffer flat_k;
    khm_buffer flat_v;
    khm_buffer req_slots;
    khm_buffer flat_token_indices;
    khm_buffer page_ids;
} khm_kv_page_write_buffers;
/* Config::num_tokens_per_page (kv_page_write.rs:76-89); 0 when page_bytes is no multiple of the K/V bytes per token. */
uint32_t khm_kv_page_write_num_tokens_per_page(const khm_kv_page_write_config* config);
/* Compute::invoke + Invocation::record (kv_page_write.rs:160-262): one launch, enqueued on `stream`. */
int khm_kv_page_write(const khm_kv_page_write_config* config, const khm_kv_page_write_shape* shape,
                      const khm_kv_page_write_buffers* buffers, khm_replay_u32 num_active_token_writes,
                      khm_replay_u32 page_table_index, const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dense bidirectional block SDPA: components/gqa/bidi_block_sdpa.rs:44-340, gqa_bidi_block_sdpa.metal:10-126
 * Every Q token attends, unmasked, to the block_size local K/V tokens of its own request block; the result is written
 * as the LAST partial state of the token's Q range (slot cu_sdpa_partial_outputs[range + 1] - 1) in the sliced-Q
 * partial layout, so that khm_sliced_q_reduce merges it with the history partials of khm_sliced_q_map.
 * ------------------------------------------------------------------------------------------ */
/* bidi_block_sdpa::Config (bidi_block_sdpa.rs:55-63). */
typedef struct khm_bidi_block_sdpa_config {
    uint32_t block_size;
    uint32_t max_q_tokens;
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    float scale;
    uint32_t dtype; /* KHM_DTYPE_F32 or KHM_DTYPE_BF16: q, local_k, local_v and partial_output */
} khm_bidi_block_sdpa_config;
/* bidi_block_sdpa::Shape (bidi_block_sdpa.rs:140-145). */
typedef struct khm_bidi_block_sdpa_shape {
    uint32_t num_total_tokens;
    uint32_t num_total_q_token_ranges;
    uint32_t num_total_partial_output_slots;
} khm_bidi_block_sdpa_shape;
/* bidi_block_sdpa::Buffers (bidi_block_sdpa.rs:175-185): q [T][Hq][D], local_k/local_v [T][Hkv][D]. */
typedef struct khm_bidi_block_sdpa_buffers {
    khm_buffer q;
    khm_buffer local_k;
    khm_buffer local_v;
    khm_buffer q_token_ranges;
    khm_buffer cu_sdpa_partial_outputs;
    khm_buffer partial_exp_sums;
    khm_buffer partial_max_logits;
    khm_buffer partial_output;
} khm_bidi_block_sdpa_buffers;
/* Compute::invoke + Invocation::record (bidi_block_sdpa.rs:227-287): one launch, enqueued on `stream`.  A Fixed
 * num_active_q_token_ranges must equal num_total_q_token_ranges, as in the reference (bidi_block_sdpa.rs:292-294).
 * head_dim must be a multiple of 32 and at most 1024 (KHM_ERR_UNSUPPORTED beyond: a lane holds at most eight
 * 8-element chunks of a Q row); the reference's Config::validate has no upper bound. */
int khm_bidi_block_sdpa(const khm_bidi_block_sdpa_config* config, const khm_bidi_block_sdpa_shape* shape,
                        const khm_bidi_block_sdpa_buffers* buffers, khm_replay_u32 num_active_q_token_ranges,
                        const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * Per-head RMSNorm + rotary embedding: components/rms_norm_rope.rs:53-403, metal/rms_norm_rope.metal:6-174
 * The step that produces the SDPA's Q (and K before the page write): out = rope(weight * x * rsqrt(mean(x^2) + eps)).
 * ------------------------------------------------------------------------------------------ */
typedef enum khm_rope_scaling_kind { KHM_ROPE_SCALING_DEFAULT = 0, KHM_ROPE_SCALING_YARN = 1 } khm_rope_scaling_kind;
/* rms_norm_rope::RopeScaling (rms_norm_rope.rs:53-64); the Yarn fields are ignored for the default kind. */
typedef struct khm_rope_scaling {
    uint32_t kind;
    float factor;
    float attention_factor;
    float beta_fast;
    float beta_slow;
    uint32_t original_max_position_embeddings;
    uint32_t truncate; /* 0 / 1 */
} khm_rope_scaling;
/* rms_norm_rope::Config (rms_norm_rope.rs:77-87). */
typedef struct khm_rms_norm_rope_config {
    uint32_t num_heads;
    uint32_t head_dim;
    uint32_t rope_dim;
    float eps;
    float rope_theta;
    khm_rope_scaling rope_scaling;
    uint32_t dtype;             /* input/output: KHM_DTYPE_F32 or KHM_DTYPE_BF16 */
    uint32_t norm_weight_dtype; /* KHM_DTYPE_F32 or KHM_DTYPE_BF16 */
} khm_rms_norm_rope_config;
/* rms_norm_rope::Buffers (rms_norm_rope.rs:286-292): input/output [T][num_heads][head_dim], norm_weight [head_dim],
 * flat_token_indices u32 [T] (the rotary positions). */
typedef struct khm_rms_norm_rope_buffers {
    khm_buffer input;
    khm_buffer norm_weight;
    khm_buffer flat_token_indices;
    khm_buffer output;
} khm_rms_norm_rope_buffers;
/* RopeScaling::yarn_kernel_parameters (rms_norm_rope.rs:206-243): the Yarn correction range (host only). */
int khm_rms_norm_rope_yarn_correction_range(const khm_rms_norm_rope_config* config, float* low, float* high);
/* RopeScaling::kernel_parameters (rms_norm_rope.rs:245-270): rope_dim / 2 inverse frequencies and the attention
 * factor (host only). */
int khm_rms_norm_rope_kernel_parameters(const khm_rms_norm_rope_config* config, float* inverse_frequencies, uint32_t capacity,
                                        float* attention_factor);
/* Compute::invoke + Invocation::record (rms_norm_rope.rs:312-384): one launch, enqueued on `stream`. */
int khm_rms_norm_rope(const khm_rms_norm_rope_config* config, uint32_t num_total_tokens, const khm_rms_norm_rope_buffers* buffers,
                      khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream);

/* K RMSNorm + RoPE fused with the K/V page write: what GQA::record enqueues as k_norm_rope -> scratch.k_norm_rope ->
 * kv_page_write (crates/inference-executor-metal/src/attn/gqa/backend.rs:382-412; rms_norm_rope.rs:286-403,
 * kv_page_write.rs:136-262) as one launch without the bf16 K round trip through memory.  The pages receive exactly the
 * bytes the two calls would have written.  norm_config.num_heads / head_dim must equal page_config.num_kv_heads /
 * head_dim and norm_config.dtype must be BF16; flat_token_indices are both the rotary positions and the token slots of
 * the writes, as in the reference.  KHM_ERR_UNSUPPORTED for shapes outside the vector path (head_dim > 512, head_dim or
 * rope_dim / 2 no multiple of 8, buffers not 16-byte aligned): the two separate calls cover those. */
typedef struct khm_k_norm_rope_page_write_buffers {
    khm_buffer pages;
    khm_buffer k;           /* bf16 [W][Hkv][D], before the norm */
    khm_buffer v;           /* bf16 [W][Hkv][D] */
    khm_buffer norm_weight; /* [D], norm_config.norm_weight_dtype */
    khm_buffer req_slots;
    khm_buffer flat_token_indices;
    khm_buffer page_ids;
} khm_k_norm_rope_page_write_buffers;
int khm_k_norm_rope_page_write(const khm_rms_norm_rope_config* norm_config, const khm_kv_page_write_config* page_config,
                               const khm_kv_page_write_shape* shape, const khm_k_norm_rope_page_write_buffers* buffers,
                               khm_replay_u32 num_active_tokens, khm_replay_u32 page_table_index,
                               const uint32_t* replay_parameters, void* stream);

/* The projection split, Q RMSNorm + RoPE, K RMSNorm + RoPE and the K/V page write as one launch: everything GQA::record
 * enqueues between the input projection and the SDPA (crates/inference-executor-metal/src/attn/gqa/backend.rs:358-412;
 * qgkv_split.rs:187-236, rms_norm_rope.rs:286-403, kv_page_write.rs:136-262), reading the projection rows once and
 * writing only what the SDPA and the gate read.  q_output, gate_output and the pages receive exactly the bytes that
 * khm_gqa_qgkv_split (gated != 0; khm_gqa_qkv_split otherwise, gate_output unused), khm_rms_norm_rope on the Q rows and
 * khm_k_norm_rope_page_write on the K and V rows would have left there.  q_norm_config.num_heads is Hq,
 * k_norm_config.num_heads is Hkv = page_config.num_kv_heads; both configs must agree in head_dim, rope_dim, rope_theta,
 * rope_scaling and norm_weight_dtype (eps may differ) and take BF16 rows.  shape.num_total_token_writes is the token
 * count of all three steps.  KHM_ERR_UNSUPPORTED outside the vector path (head_dim > 512, head_dim or rope_dim / 2 no
 * multiple of 8, buffers not 16-byte aligned): the separate calls cover those. */
typedef struct khm_gqa_projection_norm_rope_page_write_buffers {
    khm_buffer projection;    /* bf16 [T][(2 or 1) * Hq * D + 2 * Hkv * D], read only */
    khm_buffer q_norm_weight; /* [D] */
    khm_buffer k_norm_weight; /* [D] */
    khm_buffer q_output;      /* bf16 [T][Hq][D]: normalised, rotated Q rows */
    khm_buffer gate_output;   /* bf16 [T][Hq][D]: gate rows as they are (gated form) */
    khm_buffer pages;
    khm_buffer req_slots;
    khm_buffer flat_token_indices;
    khm_buffer page_ids;
} khm_gqa_projection_norm_rope_page_write_buffers;
int khm_gqa_projection_norm_rope_page_write(uint32_t gated, const khm_rms_norm_rope_config* q_norm_config,
                                            const khm_rms_norm_rope_config* k_norm_config,
                                            const khm_kv_page_write_config* page_config, const khm_kv_page_write_shape* shape,
                                            const khm_gqa_projection_norm_rope_page_write_buffers* buffers,
                                            khm_replay_u32 num_active_tokens, khm_replay_u32 page_table_index,
                                            const uint32_t* replay_parameters, void* stream);

/* ------------------------------------------------------------------------------------------
 * Executor-side host logic that feeds the component (CPU only, no HIP calls)
 * ------------------------------------------------------------------------------------------ */

/* ReplayBucketPolicy (crates/inference-executor-core/src/replay.rs:1-87). */
typedef struct khm_replay_bucket_policy khm_replay_bucket_policy;
int khm_replay_bucket_policy_create(uint32_t max_capacity, const uint32_t* topology_boundaries,
                                    uint32_t num_boundaries, khm_replay_bucket_policy** out);
void khm_replay_bucket_policy_destroy(khm_replay_bucket_policy* policy);
uint32_t khm_replay_bucket_policy_max_capacity(const khm_replay_bucket_policy* policy);
/* buckets(): copies up to `capacity` values, *count receives the total. */
int khm_replay_bucket_policy_buckets(const khm_replay_bucket_policy* policy, uint32_t* buckets, uint32_t capacity,
                                     uint32_t* count);
/* capacity(active): *out receives the bucket; errors repeat the reference panics. */
int khm_replay_bucket_policy_capacity(const khm_replay_bucket_policy* policy, uint32_t active, uint32_t* out);
int khm_replay_bucket_policy_capacity_allow_zero(const khm_replay_bucket_policy* policy, uint32_t active,
                                                 uint32_t* out);

/* RequestShape (crates/inference-executor-metal/src/attn/gqa/sdpa.rs:15-42). */
typedef struct khm_request_shape {
    uint32_t num_history_tokens;
    uint32_t num_q_tokens;
} khm_request_shape;
/* RequestShape::from_batch. */
int khm_request_shapes_from_batch(const uint32_t* token_indices, const uint32_t* cu_tokens, uint32_t num_requests,
                                  khm_request_shape* out);

/* GQAReplayShape (attn/gqa/batch_metadata.rs:11-61). */
typedef struct khm_gqa_replay_shape {
    uint32_t num_tokens;
    uint32_t num_total_tokens;
    uint32_t num_q_token_tiles;
    uint32_t num_total_q_token_tiles;
    uint32_t num_sdpa_map_task_templates;
    uint32_t num_total_sdpa_map_task_templates;
    uint32_t reduce_sdpa_partial_outputs; /* bool */
} khm_gqa_replay_shape;

/* SelectorLimits (sdpa.rs:44-49). */
typedef struct khm_selector_limits {
    uint32_t max_tokens;
    uint32_t max_map_task_templates;
    uint64_t partial_state_group_capacity;
} khm_selector_limits;

/* QTokenRange (sdpa.rs:51-57). */
typedef struct khm_q_token_range {
    uint32_t request_index;
    uint32_t flat_q_token_begin;
    uint32_t flat_q_token_end;
    uint32_t num_visible_kv_tokens;
} khm_q_token_range;

/* MapTaskTemplate (sdpa.rs:59-63). */
typedef struct khm_map_task_template {
    uint32_t q_token_range_index;
    uint32_t kv_token_begin;
    uint32_t kv_token_end;
} khm_map_task_template;

/* SelectionMetrics (sdpa.rs:65-77). */
typedef struct khm_selection_metrics {
    uint64_t num_scheduled_qk_token_pairs;
    uint64_t num_active_qk_token_pairs;
    uint64_t num_map_threadblocks_per_kv_head;
    uint64_t num_map_simdgroup_waves_per_kv_head;
    uint64_t num_active_partial_state_groups;
    uint64_t num_active_partial_states;
    uint64_t num_reserved_partial_state_groups;
    uint64_t num_replay_reserved_partial_state_groups;
    uint32_t max_kv_iterations_per_split;
    uint32_t reserved;
    uint64_t num_logical_qk_token_pairs;
} khm_selection_metrics;

typedef struct khm_selector khm_selector;   /* Selector (sdpa.rs:129-134) */
typedef struct khm_selection khm_selection; /* Selection (sdpa.rs:89-97) */

/* Selector::new over Registry::from_variants (sdpa.rs:137-163). */
int khm_selector_create(const khm_sdpa_config* config, const khm_sdpa_variant* variants, uint32_t num_variants,
                        uint64_t max_tokens, uint64_t max_map_task_templates, uint64_t partial_state_group_capacity,
                        khm_selector** out);
/* Selector::for_partitions (sdpa.rs:165-208); max_kv_splits[i] belongs to variants[i]. */
int khm_selector_create_for_partitions(const khm_sdpa_config* config, const khm_sdpa_variant* variants,
                                       const uint32_t* max_kv_splits, uint32_t num_variants, uint32_t max_tokens,
                                       uint32_t max_requests, khm_selector** out);
/* Selector::for_lookup (sdpa.rs:210-272) with the lookup table re-derived for 256 CUs. */
int khm_selector_create_for_lookup(const khm_sdpa_config* config, uint64_t max_tokens,
                                   const khm_page_table_layout* layout, khm_selector** out);
void khm_selector_destroy(khm_selector* selector);
int khm_selector_limits_get(const khm_selector* selector, khm_selector_limits* out);
int khm_selector_variants(const khm_selector* selector, khm_sdpa_variant* variants, uint32_t capacity,
                          uint32_t* count);

/* Selector::select (sdpa.rs:278-378).  The bucket policy is GQAReplayBucketPolicy::new(policy_max_tokens,
 * policy_max_map_task_templates) (batch_metadata.rs:69-96). */
int khm_selector_select(const khm_selector* selector, const khm_request_shape* request_shapes, uint32_t num_requests,
                        uint32_t policy_max_tokens, uint32_t policy_max_map_task_templates,
                        uint32_t num_total_tokens, khm_selection** out);
/* Selector::select_partitioned (sdpa.rs:380-426): explicit variant and fixed KV slice. */
int khm_selector_select_partitioned(const khm_selector* selector, const khm_sdpa_variant* variant, uint32_t kv_slice,
                                    int direct_output, const khm_request_shape* request_shapes,
                                    uint32_t num_requests, uint32_t policy_max_tokens,
                                    uint32_t policy_max_map_task_templates, uint32_t num_total_tokens,
                                    khm_selection** out);
void khm_selection_destroy(khm_selection* selection);
int khm_selection_variant(const khm_selection* selection, khm_sdpa_variant* out);
int khm_selection_direct_output(const khm_selection* selection); /* 1 / 0 */
int khm_selection_replay_shape(const khm_selection* selection, khm_gqa_replay_shape* out);
int khm_selection_metrics_get(const khm_selection* selection, khm_selection_metrics* out);
uint32_t khm_selection_num_q_token_ranges(const khm_selection* selection);
uint32_t khm_selection_num_map_task_templates(const khm_selection* selection);
int khm_selection_q_token_ranges(const khm_selection* selection, khm_q_token_range* out, uint32_t capacity);
int khm_selection_map_task_templates(const khm_selection* selection, khm_map_task_template* out, uint32_t capacity);
/* cu_partial_outputs_by_q_token_range: num_q_token_ranges + 1 values. */
int khm_selection_cu_partial_outputs(const khm_selection* selection, uint32_t* out, uint32_t capacity);

/* GQAMetadataBuffers (attn/gqa/batch_metadata.rs:98-326): capacity-sized device arrays refreshed from one
 * selection.  update() fills pinned staging memory and enqueues the host-to-device copies on `stream`
 * (the reference writes shared-memory buffers directly); arrays the reference leaves untouched stay
 * untouched (q_token_ranges for the sliced-KV kind, every tail beyond the written prefix).
 * create() and destroy() allocate and free device and pinned memory, and update() waits for `stream`: none of the three
 * may run while any stream of the process is under hipGraph capture in the global mode (the capture is invalidated and
 * its next enqueue fails).  A host language with finalizers must not leave destroy() to its collector. */
typedef struct khm_gqa_metadata khm_gqa_metadata;
typedef enum khm_gqa_metadata_array {
    KHM_METADATA_REQ_SLOTS = 0,               /* u32 [max_tokens] */
    KHM_METADATA_FLAT_TOKEN_INDICES = 1,      /* u32 [max_tokens] */
    KHM_METADATA_VISIBLE_KV_TOKEN_RANGES = 2, /* u32 [max_tokens][2] */
    KHM_METADATA_Q_TOKEN_RANGES = 3,          /* u32 [max_tokens][2] */
    KHM_METADATA_SDPA_MAP_TASK_TEMPLATES = 4, /* u32 [max_map_task_templates][3] */
    KHM_METADATA_CU_SDPA_PARTIAL_OUTPUTS = 5  /* u32 [max_tokens + 1] */
} khm_gqa_metadata_array;
int khm_gqa_metadata_create(uint64_t max_tokens, uint64_t max_map_task_templates, khm_gqa_metadata** out);
void khm_gqa_metadata_destroy(khm_gqa_metadata* metadata);
int khm_gqa_metadata_update(khm_gqa_metadata* metadata, const uint32_t* req_slots, const uint32_t* token_indices,
                            const uint32_t* cu_tokens, uint32_t num_requests, const khm_selection* selection,
                            void* stream, khm_gqa_replay_shape* out_shape);
/* Device view of one array (valid until destroy). */
int khm_gqa_metadata_buffer(const khm_gqa_metadata* metadata, uint32_t which, khm_buffer* out);
/* Host mirror of the same array (what the last update wrote; for tests and debugging). */
int khm_gqa_metadata_host(const khm_gqa_metadata* metadata, uint32_t which, const uint32_t** out, uint64_t* count);
/* Pure host form of update(): computes the uploaded prefixes into caller arrays without touching a device.
 * Each *_count receives the number of u32 values written. */
int khm_gqa_metadata_compute(const uint32_t* req_slots, const uint32_t* token_indices, const uint32_t* cu_tokens,
                             uint32_t num_requests, const khm_selection* selection, uint32_t* req_slots_by_token,
                             uint32_t* flat_token_indices, uint32_t* visible_kv_token_ranges,
                             uint32_t* q_token_ranges, uint32_t* sdpa_map_task_templates,
                             uint32_t* cu_sdpa_partial_outputs, uint64_t token_capacity, uint64_t template_capacity);

/* ------------------------------------------------------------------------------------------
 * Block (DFlash2 proposal) attention, host side: every Q-token range reduces its history split-KV partials plus one dense
 * block partial (khm_bidi_block_sdpa writes it into the last slot of the range).  Pure host logic, no device calls.
 * ------------------------------------------------------------------------------------------ */
/* BiDiBlockCapacity (inference-executor-core/src/attn/gqa/bidi_block_gqa_core.rs:27-63) + BiDiBlockGQACapacity
 * (inference-executor-metal/src/attn/bidi_block_gqa/capacity.rs:7-48). */
typedef struct khm_bidi_block_capacity {
    uint32_t max_requests;
    uint32_t block_size;
    uint32_t max_tokens;
    uint32_t max_q_tokens;
    uint32_t max_q_token_ranges;
    uint32_t max_sdpa_map_task_templates;
    uint64_t max_sdpa_partial_state_groups;
} khm_bidi_block_capacity;
int khm_bidi_block_capacity_new(uint32_t max_requests, uint32_t block_size, uint32_t max_q_tokens, khm_bidi_block_capacity* out);
/* bidi_block_gqa::sdpa::Selector::select (attn/bidi_block_gqa/sdpa.rs:46-110): the registry variant that loads the
 * history K/V least often for a fixed block width, and the capacity that goes with it. */
int khm_bidi_block_select(const khm_sdpa_config* config, uint32_t max_requests, uint32_t block_size, khm_sdpa_variant* variant,
                          khm_bidi_block_capacity* capacity);
/* BiDiBlockGQAMetadata::new (bidi_block_gqa_core.rs:77-139) + build_metal_metadata and
 * BiDiBlockGQAMetadataBuffers::update_with_active_requests (attn/bidi_block_gqa/metadata.rs:87-147,182-375).
 * Inputs: req_slots [R] (unique), and per block row (R * block_size rows) the query token index and its nonempty visible
 * history range.  Outputs (host arrays): req_slots_by_token / flat_token_indices [T], visible_kv_token_ranges [T][2],
 * q_token_ranges [ranges][2], sdpa_map_task_templates [max_sdpa_map_task_templates][3] (written up to the replay
 * capacity, padded with u32::MAX; each range's last template is the u32::MAX placeholder of its block partial),
 * cu_sdpa_partial_outputs [ranges + 1], and the replay shape of the first num_active_requests requests. */
int khm_bidi_block_metadata_compute(const uint32_t* req_slots, uint32_t num_requests, const uint32_t* flat_query_token_indices,
                                    const uint32_t* history_token_begins, const uint32_t* history_token_ends, uint32_t block_size,
                                    const khm_sdpa_variant* variant, uint32_t max_sdpa_map_task_templates,
                                    uint32_t num_active_requests, uint32_t* req_slots_by_token, uint32_t* flat_token_indices,
                                    uint32_t* visible_kv_token_ranges, uint32_t* q_token_ranges, uint32_t* sdpa_map_task_templates,
                                    uint32_t* cu_sdpa_partial_outputs, khm_gqa_replay_shape* out_shape);

#ifdef __cplusplus
}
#endif
#endif /* KHM_GQA_SDPA_H */
