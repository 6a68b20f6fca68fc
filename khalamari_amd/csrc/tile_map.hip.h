// Tiled Map kernel for chunked prefill and wide verify blocks on gfx950 (bf16 MFMA, LDS-shared K/V tiles).
//
// Replaces gqa_sdpa_sliced_q_map / gqa_sdpa_sliced_q_per_head_map for Q tiles above 64 coordinates
// (crates/inference-backend-metal/src/components/metal/gqa_sdpa_sliced_q_map.metal:29-284,
// gqa_sdpa_sliced_q_per_head_map.metal:25-298): same task ABI (one block per map task template x KV head x
// Q-head range), same per-token visible range mask, same partial-state contract, and the direct-output mode.
//
// Work shape.  A block owns up to NWAVES * NTW * 16 (q_token, q_head) columns; each wave owns NTW 16-column
// tiles for the whole KV range, so there is no cross-wave merge.  KV is walked in BK-token tiles that all
// waves share through LDS.  Per tile and wave:
//     S^T[BK][cols] = K . Q^T        v_mfma_f32_16x16x32_bf16, K rows (ds_read_b128) as the A operand, Q in registers
//     online softmax per column      exp2 domain; the accumulator is rescaled only when a column's maximum moved
//     O^T[D][cols] += V^T . P^T      v_mfma_f32_16x16x32_bf16; the V^T operand comes from row-major V in LDS through
//                                    ds_read_b64_tr_b16 (each lane receives 4 tokens of one dim), P stays in registers
// Memory.  The block loads tile i+2 from HBM (fully coalesced 16-byte chunks, one 16-token page slab per pass)
// into registers while it computes tile i; LDS is double-buffered so one barrier per tile suffices.
// Blocks are renumbered so that each XCD walks a contiguous run of the (KV head, template) list: the Q ranges of
// one sequence share their K/V through that XCD's L2 instead of each pulling it from HBM.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.hip.h"
#include "device_params.h"

namespace khm {

typedef short s16x4v __attribute__((ext_vector_type(4)));

template <int D, int BK>
struct TileSmem {
    static constexpr int kRowBytes = D * 2 + 32;   // 32 B pad: conflict-light b128 and transposed reads
    static constexpr int kTileBytes = BK * kRowBytes;
    static constexpr int kBytes = 2 /*K,V*/ * 2 /*stages*/ * kTileBytes;
};

// LDS transpose read: lane r of every 16-lane group passes the address of 4 consecutive bf16; lane i receives
// element (i % 4) of the rows given by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 of its group.
__device__ __forceinline__ s16x4v lds_read_tr16(const unsigned char* address) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4v __attribute__((address_space(3)))*)(address));
}

template <int D, int NTW, int NWAVES, int BK>
__global__ __launch_bounds__(NWAVES * 64) void tile_map_kernel(const MapParams p) {
    constexpr int THREADS = NWAVES * 64;
    constexpr int KS = D / 32;                      // QK k-steps
    constexpr int MT = D / 16;                      // PV dim tiles
    constexpr int RT = BK / 16;                     // 16-token row tiles per KV tile
    constexpr int CHUNKS_PER_ROW = D / 8;           // 16-byte chunks per K/V row
    constexpr int ROWS_PER_PASS = THREADS / CHUNKS_PER_ROW;
    constexpr int PASSES = BK / ROWS_PER_PASS;      // global->LDS passes per plane
    static_assert(ROWS_PER_PASS <= 16 && 16 % ROWS_PER_PASS == 0, "a load pass must stay inside one 16-token group");
    static_assert(BK % 32 == 0, "PV consumes 32 tokens per MFMA");
    using Smem = TileSmem<D, BK>;

    extern __shared__ __align__(16) unsigned char tile_smem[];
    unsigned char* k_lds = tile_smem;                              // [2][BK][kRowBytes]
    unsigned char* v_lds = tile_smem + 2 * Smem::kTileBytes;       // [2][BK][kRowBytes]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;
    const int g = lane >> 4;

    // ---- XCD-aware block renumbering -------------------------------------------------------------------
    // Hardware deals consecutive block ids round-robin to the 8 XCDs.  Work item w = (head group, template)
    // in head-group-major order; XCD x takes the contiguous run [x * N / 8, (x + 1) * N / 8).
    const uint32_t num_tasks = gridDim.x;
    const uint32_t num_head_groups = gridDim.y;
    const uint64_t total = (uint64_t)num_tasks * num_head_groups;
    const uint64_t linear = (uint64_t)blockIdx.y * num_tasks + blockIdx.x;
    uint64_t work = linear;
    {
        const uint64_t per_xcd = total / 8;
        const uint64_t main = per_xcd * 8;
        if (linear < main) work = (linear % 8) * per_xcd + linear / 8;
    }
    const uint32_t head_group = (uint32_t)(work / num_tasks);
    const uint32_t task = (uint32_t)(work % num_tasks);

    // ---- task decode (uniform) ---------------------------------------------------------------------------
    if (task >= resolve_u32(p.num_active_kv_splits, p.replay_parameters)) return;
    const uint32_t range_index = p.templates[3 * (uint64_t)task];
    if (range_index >= resolve_u32(p.num_active_q_token_tiles, p.replay_parameters)) return;
    const uint32_t flat_begin = p.q_token_ranges[2 * (uint64_t)range_index];
    const uint32_t flat_end = p.q_token_ranges[2 * (uint64_t)range_index + 1];
    const uint32_t num_active_tokens = resolve_u32(p.num_active_tokens, p.replay_parameters);
    if (flat_begin >= num_active_tokens || flat_end > num_active_tokens || flat_end <= flat_begin) return;
    uint32_t num_q = flat_end - flat_begin;
    if (num_q > p.max_q_tokens) num_q = p.max_q_tokens;
    const uint32_t kv_begin = p.templates[3 * (uint64_t)task + 1];
    const uint32_t kv_end = p.templates[3 * (uint64_t)task + 2];
    const uint32_t req_slot = p.req_slots[flat_begin];
    const uint32_t layer = resolve_u32(p.layer_index, p.replay_parameters);

    const uint32_t head_range = head_group % p.num_q_head_ranges;
    const uint32_t kv_head = head_group / p.num_q_head_ranges;
    const uint32_t head_range_begin = head_range * p.max_q_heads;
    const uint32_t heads_left = p.q_heads_per_kv_head - head_range_begin;
    const uint32_t num_heads = heads_left < p.max_q_heads ? heads_left : p.max_q_heads;
    const uint32_t first_q_head = kv_head * p.q_heads_per_kv_head + head_range_begin;

    // ---- per-lane column facts ---------------------------------------------------------------------------
    uint32_t col_lo[NTW], col_hi[NTW], col_token[NTW], col_head[NTW];
    bool col_active[NTW];
    uint32_t blk_lo = 0xffffffffu, blk_hi = 0u, wave_all_lo = 0u, wave_all_hi = 0xffffffffu, min_span = 0xffffffffu;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        const uint32_t c = (wave * NTW + nt) * 16 + r16;
        const uint32_t token_offset = c / p.max_q_heads;
        const uint32_t local_head = c - token_offset * p.max_q_heads;
        col_active[nt] = token_offset < num_q && local_head < num_heads;
        col_token[nt] = token_offset;
        col_head[nt] = local_head;
        uint32_t lo = kv_begin, hi = kv_end;
        if (col_active[nt]) {
            const uint64_t token = flat_begin + token_offset;
            const uint32_t vis_lo = p.visible_ranges[2 * token];
            const uint32_t vis_hi = p.visible_ranges[2 * token + 1];
            lo = vis_lo > lo ? vis_lo : lo;
            hi = vis_hi < hi ? vis_hi : hi;
        }
        if (hi < lo) hi = lo;
        col_lo[nt] = lo;
        col_hi[nt] = hi;
        if (col_active[nt]) {
            if (hi > lo) {
                blk_lo = lo < blk_lo ? lo : blk_lo;
                blk_hi = hi > blk_hi ? hi : blk_hi;
            }
            wave_all_lo = lo > wave_all_lo ? lo : wave_all_lo;
            wave_all_hi = hi < wave_all_hi ? hi : wave_all_hi;
            min_span = hi - lo < min_span ? hi - lo : min_span;
        }
    }
#pragma unroll
    for (int offset = 1; offset < 16; offset <<= 1) {
        uint32_t other;
        other = __shfl_xor(blk_lo, offset); blk_lo = other < blk_lo ? other : blk_lo;
        other = __shfl_xor(blk_hi, offset); blk_hi = other > blk_hi ? other : blk_hi;
        other = __shfl_xor(wave_all_lo, offset); wave_all_lo = other > wave_all_lo ? other : wave_all_lo;
        other = __shfl_xor(wave_all_hi, offset); wave_all_hi = other < wave_all_hi ? other : wave_all_hi;
        other = __shfl_xor(min_span, offset); min_span = other < min_span ? other : min_span;
    }
    // Rounding a softmax weight to bf16 costs up to 2^-9 of that weight; with few keys the weights are O(1) and
    // the error shows at the 1e-3 level.  Waves whose columns see at most kPreciseSpan keys therefore feed the second
    // MFMA with hi + lo bf16 pairs (the reference keeps P in f32); long contexts, where every weight is small, use one.
    constexpr uint32_t kPreciseSpan = 256;
    const bool precise = __builtin_amdgcn_readfirstlane(min_span) <= kPreciseSpan;
    wave_all_lo = __builtin_amdgcn_readfirstlane(wave_all_lo);
    wave_all_hi = __builtin_amdgcn_readfirstlane(wave_all_hi);
    // block-wide KV range: reduce the per-wave ranges through LDS
    uint32_t* range_lds = reinterpret_cast<uint32_t*>(tile_smem);
    if (lane == 0) {
        range_lds[wave * 2] = blk_lo;
        range_lds[wave * 2 + 1] = blk_hi;
    }
    __syncthreads();
    const uint32_t wave_lo = __builtin_amdgcn_readfirstlane(blk_lo);
    const uint32_t wave_hi = __builtin_amdgcn_readfirstlane(blk_hi);
    blk_lo = 0xffffffffu;
    blk_hi = 0u;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) {
        const uint32_t lo = range_lds[w * 2], hi = range_lds[w * 2 + 1];
        blk_lo = lo < blk_lo ? lo : blk_lo;
        blk_hi = hi > blk_hi ? hi : blk_hi;
    }
    blk_lo = __builtin_amdgcn_readfirstlane(blk_lo);
    blk_hi = __builtin_amdgcn_readfirstlane(blk_hi);
    __syncthreads();
    {
        const uint64_t table_tokens = (uint64_t)p.pages_per_request_layer << p.tokens_per_page_shift;
        if (blk_hi > table_tokens) blk_hi = (uint32_t)table_tokens;
    }

    // ---- Q fragments in registers: B operand, lane holds Q[col = lane & 15][dims ks*32 + g*8 .. +8] ------------
    uint4 q_frag[NTW][KS];
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q_frag[nt][ks] = make_uint4(0, 0, 0, 0);
        if (col_active[nt]) {
            const uint16_t* row = p.q + ((uint64_t)(flat_begin + col_token[nt]) * p.num_q_heads + first_q_head + col_head[nt]) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) q_frag[nt][ks] = *reinterpret_cast<const uint4*>(row + ks * 32 + g * 8);
        }
    }

    // ---- tile schedule -------------------------------------------------------------------------------------
    const uint32_t first_group = blk_lo >> 4;                                   // 16-token groups
    const uint32_t num_groups = blk_hi > blk_lo ? ((blk_hi - 1) >> 4) - first_group + 1 : 0;
    const uint32_t num_tiles = (num_groups + RT - 1) / RT;
    const uint32_t* table = p.page_ids + ((uint64_t)req_slot * p.num_gqa_layers + layer) * p.pages_per_request_layer;
    const uint32_t tpp = p.tokens_per_page;
    const uint32_t tpp_shift = p.tokens_per_page_shift;
    const uint64_t plane_k = ((uint64_t)kv_head * tpp) * (D * 2);
    const uint64_t plane_v = ((uint64_t)(p.num_kv_heads + kv_head) * tpp) * (D * 2);

    // Page ids of 64 consecutive 16-token groups per register pair; two pairs alternate.
    uint32_t ids_a[2] = {0, 0}, ids_b[2] = {0, 0};
    auto load_ids = [&](uint32_t chunk, uint32_t (&ids)[2]) {
        const uint32_t group = chunk * 64 + lane;
        if (group < num_groups) {
            const uint32_t token = (first_group + group) << 4;
            const uint32_t last_page = p.pages_per_request_layer - 1;
            const uint32_t page0 = token >> tpp_shift;
            const uint32_t page1 = (token + 8) >> tpp_shift;
            ids[0] = table[page0 < last_page ? page0 : last_page];
            ids[1] = table[page1 < last_page ? page1 : last_page];
        }
    };
    load_ids(0, ids_a);
    if (num_groups > 64) load_ids(1, ids_b);

    uint4 stage_k[PASSES], stage_v[PASSES];
    const uint32_t load_row = tid / CHUNKS_PER_ROW;    // row inside a pass
    const uint32_t load_chunk = tid % CHUNKS_PER_ROW;
    auto load_tile = [&](uint32_t tile) {
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const uint32_t row = pass * ROWS_PER_PASS + load_row;                // row inside the tile
            uint32_t group = tile * RT + (row >> 4);
            if (group >= num_groups) group = num_groups - 1;                     // tail rows: any valid page, masked below
            const uint32_t chunk = group >> 6;
            const uint32_t sel0 = (chunk & 1) ? ids_b[0] : ids_a[0];
            const uint32_t sel1 = (chunk & 1) ? ids_b[1] : ids_a[1];
            uint32_t id0 = __builtin_amdgcn_readlane(sel0, group & 63);
            uint32_t id1 = __builtin_amdgcn_readlane(sel1, group & 63);
            const uint32_t first_token = (first_group + group) << 4;
            if (tpp == 8) {
                if (first_token + 8 >= blk_hi) id1 = id0;
                if (first_token + 8 <= blk_lo) id0 = id1;
            }
            const uint32_t row16 = row & 15;
            const uint32_t in_page = (first_token + row16) & (tpp - 1);
            const uint64_t page = row16 >= 8 ? id1 : id0;
            const unsigned char* base = p.kv_pages + page * p.page_bytes + (uint64_t)in_page * (D * 2) + load_chunk * 16;
            stage_k[pass] = *reinterpret_cast<const uint4*>(base + plane_k);
            stage_v[pass] = *reinterpret_cast<const uint4*>(base + plane_v);
        }
    };
    auto refresh_ids = [&](uint32_t tile) {
        // Called once per tile by every wave (uniform): when the tile starts a new 64-group id chunk, prefetch the next one.
        const uint32_t group = tile * RT;
        const uint32_t chunk = group >> 6;
        if ((group & 63) < (uint32_t)RT && chunk >= 1 && (chunk + 1) * 64 < num_groups) {
            if ((chunk + 1) & 1) load_ids(chunk + 1, ids_b); else load_ids(chunk + 1, ids_a);
        }
    };
    auto store_tile = [&](uint32_t tile, int stage) {
        unsigned char* k_dst = k_lds + stage * Smem::kTileBytes;
        unsigned char* v_dst = v_lds + stage * Smem::kTileBytes;
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const uint32_t row = pass * ROWS_PER_PASS + load_row;
            const uint32_t token = ((first_group + tile * RT) << 4) + row;
            uint4 v = stage_v[pass];
            if (token < blk_lo || token >= blk_hi) v = make_uint4(0, 0, 0, 0);  // unused page slots may hold anything
            *reinterpret_cast<uint4*>(k_dst + row * Smem::kRowBytes + load_chunk * 16) = stage_k[pass];
            *reinterpret_cast<uint4*>(v_dst + row * Smem::kRowBytes + load_chunk * 16) = v;
        }
    };

    // ---- online-softmax state ------------------------------------------------------------------------------
    f32x4 acc[NTW][MT];
    float run_max[NTW], run_sum[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        run_max[nt] = -INFINITY;
        run_sum[nt] = 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    auto compute_tile = [&](uint32_t tile, int stage) {
        const uint32_t tile_first = (first_group + tile * RT) << 4;
        // Tiles entirely outside this wave's own columns' ranges contribute nothing (causal skew inside the block).
        if (tile_first >= wave_hi || tile_first + BK <= wave_lo) return;
        const unsigned char* k_src = k_lds + stage * Smem::kTileBytes;
        const unsigned char* v_src = v_lds + stage * Smem::kTileBytes;
        f32x4 s[RT][NTW];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) s[rt][nt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const uint4 a_bits = *reinterpret_cast<const uint4*>(k_src + (rt * 16 + r16) * Smem::kRowBytes + (ks * 32 + g * 8) * 2);
                const bf16x8 a = __builtin_bit_cast(bf16x8, a_bits);
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt)
                    s[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, q_frag[nt][ks]), s[rt][nt], 0, 0, 0);
            }
        }
        const bool interior = tile_first >= wave_all_lo && tile_first + BK <= wave_all_hi;
        uint32_t p_bits[RT][NTW][2], p_low[RT][NTW][2];
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            float tile_max = -INFINITY;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v = s[rt][nt][i];
                    if (!interior) {
                        const uint32_t token = tile_first + rt * 16 + g * 4 + i;
                        v = (token >= col_lo[nt] && token < col_hi[nt]) ? v : -INFINITY;
                        s[rt][nt][i] = v;
                    }
                    tile_max = fmaxf(tile_max, v);
                }
            }
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
            tile_max *= p.scale_log2e;                                 // scale > 0: max commutes with the scaling
            const float next_max = fmaxf(run_max[nt], tile_max);
            const float safe_max = next_max == -INFINITY ? 0.0f : next_max;
            const float alpha = fast_exp2(run_max[nt] - safe_max);
            run_max[nt] = next_max;
            float tile_sum = 0.0f;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                float e[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    e[i] = fast_exp2(__builtin_fmaf(s[rt][nt][i], p.scale_log2e, -safe_max));
                    tile_sum += e[i];
                }
                p_bits[rt][nt][0] = pack_bf16x2(e[0], e[1]);
                p_bits[rt][nt][1] = pack_bf16x2(e[2], e[3]);
                if (precise) {
                    p_low[rt][nt][0] = pack_bf16x2(e[0] - bf16_bits_to_f32(p_bits[rt][nt][0] & 0xffffu), e[1] - bf16_bits_to_f32(p_bits[rt][nt][0] >> 16));
                    p_low[rt][nt][1] = pack_bf16x2(e[2] - bf16_bits_to_f32(p_bits[rt][nt][1] & 0xffffu), e[3] - bf16_bits_to_f32(p_bits[rt][nt][1] >> 16));
                }
            }
            run_sum[nt] = run_sum[nt] * alpha + tile_sum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[nt][mt] *= alpha;
            }
        }
        // O^T += V^T . P^T, 32 tokens per MFMA: k = 8g + j <-> token (j < 4 ? 4g + j : 16 + 4g + j - 4) of the 32-token pair.
#pragma unroll
        for (int pair = 0; pair < RT / 2; ++pair) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const unsigned char* column = v_src + (pair * 32 + g * 4 + (r16 >> 2)) * Smem::kRowBytes + (mt * 16 + (r16 & 3) * 4) * 2;
                const s16x4v lo = lds_read_tr16(column);
                const s16x4v hi = lds_read_tr16(column + 16 * Smem::kRowBytes);
                const uint4 a_bits = make_uint4(__builtin_bit_cast(uint2, lo).x, __builtin_bit_cast(uint2, lo).y,
                                                __builtin_bit_cast(uint2, hi).x, __builtin_bit_cast(uint2, hi).y);
                const bf16x8 a = __builtin_bit_cast(bf16x8, a_bits);
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) {
                    const uint4 b_bits = make_uint4(p_bits[2 * pair][nt][0], p_bits[2 * pair][nt][1], p_bits[2 * pair + 1][nt][0],
                                                    p_bits[2 * pair + 1][nt][1]);
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, b_bits), acc[nt][mt], 0, 0, 0);
                    if (precise) {
                        const uint4 low_bits = make_uint4(p_low[2 * pair][nt][0], p_low[2 * pair][nt][1], p_low[2 * pair + 1][nt][0],
                                                          p_low[2 * pair + 1][nt][1]);
                        acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, low_bits), acc[nt][mt], 0, 0, 0);
                    }
                }
            }
        }
    };

    // ---- main loop: registers hold tile i+1 while LDS stage i%2 is consumed -------------------------------------
    if (num_tiles > 0) {
        load_tile(0);
        store_tile(0, 0);
        if (num_tiles > 1) load_tile(1);
        for (uint32_t tile = 0; tile < num_tiles; ++tile) {
            __syncthreads();  // stage tile%2 is complete; nobody still reads stage (tile+1)%2
            if (tile + 1 < num_tiles) store_tile(tile + 1, (tile + 1) & 1);
            if (tile + 2 < num_tiles) {
                refresh_ids(tile + 2);
                load_tile(tile + 2);
            }
            compute_tile(tile, tile & 1);
        }
    }

    // ---- epilogue: every wave owns its columns, no cross-wave merge ------------------------------------------------
    const uint32_t mode = p.output_mode;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        float total = run_sum[nt];
        total += __shfl_xor(total, 16);
        total += __shfl_xor(total, 32);
        if (!col_active[nt]) continue;
        const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
        const uint32_t q_head = first_q_head + col_head[nt];
        uint64_t row;
        if (mode == kMapDirectBf16) {
            row = (uint64_t)(flat_begin + col_token[nt]) * p.num_q_heads + q_head;
        } else {
            row = ((uint64_t)task * p.num_q_heads + q_head) * p.max_q_tokens + col_token[nt];
            if (g == 0) {
                p.exp_sums[row] = total;
                p.max_logits[row] = total > 0.0f ? run_max[nt] * 0.6931471805599453f : -INFINITY;
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const f32x4 value = acc[nt][mt] * inverse;
            const uint32_t d = mt * 16 + g * 4;
            if (mode == kMapPartialF32) {
                *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.out) + row * D + d) = value;
            } else {
                const uint2 packed = make_uint2(pack_bf16x2(value[0], value[1]), pack_bf16x2(value[2], value[3]));
                *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.out) + row * D + d) = packed;
            }
        }
    }
}

}  // namespace khm
