// Split-KV Map kernel for decode and speculative-verify blocks on gfx950 (wave64, bf16 MFMA).
//
// Replaces gqa_sdpa_sliced_kv_map (crates/inference-backend-metal/src/components/metal/
// gqa_sdpa_sliced_kv_map.metal:36-211) and, for small Q tiles, gqa_sdpa_sliced_q_map
// (.../gqa_sdpa_sliced_q_map.metal:29-284).  Same task ABI: one block per
// (map task template, KV head, Q-head range); same partial-state contract: normalized partial,
// exp-sum, natural-log max, canonical empty state (0, -inf, 0), inactive coordinates untouched.
//
// Work shape.  The block's Q coordinates (q_token, q_head) are the N columns of 16-wide MFMA
// tiles (NT tiles).  KV is walked in 16-token tiles; wave w of the block takes tiles
// w, w + NWAVES, ...  Per tile a wave computes
//     S^T[token][col] = K[token][:] . Q[col][:]           v_mfma_f32_16x16x32_bf16, K as the A operand
//     online softmax per column (exp2 domain, f32)
//     O^T[dim][col]  += V^T[dim][token] . P^T[token][col]  v_mfma_f32_16x16x16_bf16
// Computing S transposed makes the softmax weights land in exactly the register layout the
// second MFMA wants for its B operand, so P never moves between lanes, and the per-column
// rescale factor is a per-lane scalar.
//
// Memory.  K rows go from HBM straight into the A-operand layout (each lane: one token row,
// 16 B per k-step).  V rows are loaded as fully coalesced 16-byte chunks, written to a
// wave-private LDS tile and read back transposed (4 tokens of one dim per lane).  Loads for
// tile j+2 are issued before tile j is consumed (three register buffers).  Page ids are read
// once per 64 tiles into a register and broadcast with v_readlane, so the page-table lookup is
// never on the critical path of a K/V load.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.hip.h"
#include "device_params.h"
#include "fp8_device.hip.h"
#include "lse_merge.hip.h"

namespace khm {

// One 16-token K/V tile in registers, 16 bytes per lane and load.
//   bf16 pages: k[ks] is the A-operand fragment of k-step ks: token row (lane & 15), dims ks*32 + (lane >> 4)*8 .. +8;
//               v[i] is a coalesced chunk: row i*(512/D) + lane/(D/8), dims (lane % (D/8))*8 .. +8.
//   FP8 pages:  16 bytes are 16 dims, so k[j] feeds two k-steps: token row (lane & 15), dims j*64 + (lane >> 4)*16 .. +16,
//               the low eight for k-step 2j and the high eight for k-step 2j+1 (the Q operand uses the same dim order);
//               v[i] is row i*(1024/D) + lane/(D/16), dims (lane % (D/16))*16 .. +16.
template <int D, bool KV8>
struct KvTile {
    static constexpr int kLoads = KV8 ? D / 64 : D / 32;
    uint4 k[kLoads];
    uint4 v[kLoads];
    uint32_t first_token;
};

template <int D, int NT, int NWAVES, bool Q_IN_LDS = (NT != 1)>
struct MapSmem {
    static constexpr int kVRowBytes = D * 2 + 32;          // +32 B: rows 8 banks apart, conflict-free transposed reads
    static constexpr int kVBytes = NWAVES * 16 * kVRowBytes;
    static constexpr int kCols = NT * 16;
    static constexpr int kORowFloats = D + 4;
    // one merged tile, or (one column tile) a tile per wave so that all waves hand over their accumulators at once
    static constexpr bool kTilePerWave = (NT == 1);
    static constexpr int kOBytes = (kTilePerWave ? NWAVES : 1) * kCols * kORowFloats * 4;
    static constexpr int kUnionBytes = kVBytes > kOBytes ? kVBytes : kOBytes;
    static constexpr int kQRowBytes = D * 2 + 16;
    static constexpr int kQBytes = Q_IN_LDS ? kCols * kQRowBytes : 0;   // a single column tile keeps Q in registers
    static constexpr int kStatsBytes = (NWAVES + 1) * kCols * 3 * 4;   // (reference, sum, maximum) per wave and column
    static constexpr int kTotal = kUnionBytes + kQBytes + kStatsBytes;
};

// K/V tiles requested ahead of the one being consumed (register buffers: one more than this).
constexpr int kMapPrefetchDepth = 2;

template <int D, int NT, int NWAVES, bool KV8 = false>
__global__ __launch_bounds__(NWAVES * 64) void split_kv_map_kernel(const MapParams p) {
    constexpr int KS = D / 32;
    constexpr int MT = D / 16;
    constexpr int COLS = NT * 16;
    constexpr int ELEMENT_BYTES = KV8 ? 1 : 2;    // K/V page element: FP8 E4M3FN or bf16
    constexpr int ROW_BYTES = D * ELEMENT_BYTES;
    constexpr int LANES_PER_ROW = ROW_BYTES / 16; // 16-byte chunks per K/V row
    constexpr int ROWS_PER_LOAD = 64 / LANES_PER_ROW;
    constexpr int LOADS = KvTile<D, KV8>::kLoads;
    // first dim of the eight that lane group g contracts in k-step ks (the K fragments above fix the order)
    auto q_dim = [](int ks, int g) { return KV8 ? (ks >> 1) * 64 + g * 16 + (ks & 1) * 8 : ks * 32 + g * 8; };
    // D 256 on FP8 pages: with the Q fragments read from LDS and one tile requested ahead instead of two the kernel takes
    // 236 registers instead of 296, so a compute unit holds two blocks (two waves per SIMD) instead of one; these blocks
    // run at the pace of their own load -> decode -> MFMA chain, which a second wave on the SIMD overlaps (four requests of
    // 131072 tokens: 200 -> 194 us).  bf16 pages at D 256 stay at one block either way (399 registers) and are within 3 %
    // of a read-only launch; at D 128 a third block per CU was measured and changes nothing.
    constexpr bool kSlim = D == 256 && KV8;
    constexpr bool kQInRegs = (NT == 1) && !kSlim;
    using Smem = MapSmem<D, NT, NWAVES, !kQInRegs>;

    __shared__ __align__(16) unsigned char smem[Smem::kTotal];
    unsigned char* v_lds_all = smem;
    float* o_lds = reinterpret_cast<float*>(smem);
    unsigned char* q_lds = smem + Smem::kUnionBytes;
    float* stats_lds = reinterpret_cast<float*>(smem + Smem::kUnionBytes + Smem::kQBytes);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;
    const int g = lane >> 4;

    // ---- task decode (uniform) -------------------------------------------------------------
    // Blocks are dispatched in linear order; the KV heads of one task vary fastest, so the blocks in flight together
    // read neighbouring slabs of the same pages (a whole 64 KB page between the eight heads) instead of the same
    // 4 KB window of many pages, which spreads the requests evenly over the memory channels (+4 % on config 2).
    const uint32_t linear_block = blockIdx.y * gridDim.x + blockIdx.x;
    const uint32_t task = linear_block / gridDim.y;
    const uint32_t head_group_index = linear_block % gridDim.y;
    // The metadata chain in front of a block's first K/V load is a chain of dependent round trips to memory, a fifth of
    // the life of a 512-token decode block: arguments -> task template -> request slot -> page ids -> K/V.  Every link is
    // a scalar load, and everything that hangs on the same link is requested together: the whole argument block; then
    // the template's three words and the replay values; then (sliced-Q) the Q range; then the request slot.  The grid
    // has one block per template of the padded shape, so reading the template before the activity test is in bounds.
    fetch_all_arguments(p);
    const ReplayValues replay = resolve_replay_values(p);
    const uint32_t range_index = load_uniform_u32(p.templates, 3 * (uint64_t)task);
    const uint32_t kv_begin = load_uniform_u32(p.templates, 3 * (uint64_t)task + 1);
    const uint32_t kv_end = load_uniform_u32(p.templates, 3 * (uint64_t)task + 2);
    const uint32_t num_active_splits = replay.num_active_kv_splits;
    if (task >= num_active_splits) return;
    if (range_index >= replay.num_active_q_token_tiles) return;
    uint32_t flat_begin, flat_end;
    if (p.q_token_ranges != nullptr) {
        flat_begin = load_uniform_u32(p.q_token_ranges, 2 * (uint64_t)range_index);
        flat_end = load_uniform_u32(p.q_token_ranges, 2 * (uint64_t)range_index + 1);
    } else {
        flat_begin = range_index;
        flat_end = range_index + 1;
    }
    const uint32_t num_active_tokens = replay.num_active_tokens;
    if (flat_begin >= num_active_tokens || flat_end > num_active_tokens || flat_end <= flat_begin) return;
    uint32_t num_q = flat_end - flat_begin;
    if (num_q > p.max_q_tokens) num_q = p.max_q_tokens;
    const uint32_t req_slot = load_uniform_u32(p.req_slots, flat_begin);
    const uint32_t layer = replay.layer;

    const uint32_t head_range = head_group_index % p.num_q_head_ranges;
    const uint32_t kv_head = head_group_index / p.num_q_head_ranges;
    const uint32_t head_range_begin = head_range * p.max_q_heads;
    const uint32_t heads_left = p.q_heads_per_kv_head - head_range_begin;
    const uint32_t num_heads = heads_left < p.max_q_heads ? heads_left : p.max_q_heads;
    const uint32_t first_q_head = kv_head * p.q_heads_per_kv_head + head_range_begin;

    // ---- per-lane column facts -------------------------------------------------------------
    // Column c = token_offset * max_q_heads + local_head.
    uint32_t col_lo[NT], col_hi[NT];
    bool col_active[NT];
    uint32_t blk_lo = 0xffffffffu, blk_hi = 0u, all_lo = 0u, all_hi = 0xffffffffu;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t c = nt * 16 + r16;
        const uint32_t token_offset = c / p.max_q_heads;
        const uint32_t local_head = c - token_offset * p.max_q_heads;
        col_active[nt] = token_offset < num_q && local_head < num_heads;
        uint32_t lo = kv_begin, hi = kv_end;
        if (col_active[nt] && p.visible_ranges != nullptr) {
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
            all_lo = lo > all_lo ? lo : all_lo;
            all_hi = hi < all_hi ? hi : all_hi;
        }
    }
#pragma unroll
    for (int offset = 1; offset < 16; offset <<= 1) {
        uint32_t other;
        other = __shfl_xor(blk_lo, offset); blk_lo = other < blk_lo ? other : blk_lo;
        other = __shfl_xor(blk_hi, offset); blk_hi = other > blk_hi ? other : blk_hi;
        other = __shfl_xor(all_lo, offset); all_lo = other > all_lo ? other : all_lo;
        other = __shfl_xor(all_hi, offset); all_hi = other < all_hi ? other : all_hi;
    }
    blk_lo = __builtin_amdgcn_readfirstlane(blk_lo);
    blk_hi = __builtin_amdgcn_readfirstlane(blk_hi);
    all_lo = __builtin_amdgcn_readfirstlane(all_lo);
    all_hi = __builtin_amdgcn_readfirstlane(all_hi);
    {
        // Never walk past the request's page table.
        const uint64_t table_tokens = (uint64_t)p.pages_per_request_layer << p.tokens_per_page_shift;
        if (blk_hi > table_tokens) blk_hi = (uint32_t)table_tokens;
    }

    // ---- Q fragments -----------------------------------------------------------------------
    // B operand of S^T = K.Q^T: lane holds Q[col = lane & 15][dims ks*32 + g*8 .. +8].
    uint4 q_frag[kQInRegs ? KS : 1];
    if constexpr (kQInRegs) {
        const uint32_t c = r16;
        const uint32_t token_offset = c / p.max_q_heads;
        const uint32_t local_head = c - token_offset * p.max_q_heads;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q_frag[ks] = make_uint4(0, 0, 0, 0);
        if (col_active[0]) {
            const uint16_t* row = p.q + ((uint64_t)(flat_begin + token_offset) * p.num_q_heads + first_q_head + local_head) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) q_frag[ks] = *reinterpret_cast<const uint4*>(row + q_dim(ks, g));
        }
    } else {
        constexpr int Q_CHUNKS = D / 8;
        for (int index = tid; index < COLS * Q_CHUNKS; index += NWAVES * 64) {
            const uint32_t c = index / Q_CHUNKS;
            const uint32_t chunk = index - c * Q_CHUNKS;
            const uint32_t token_offset = c / p.max_q_heads;
            const uint32_t local_head = c - token_offset * p.max_q_heads;
            uint4 value = make_uint4(0, 0, 0, 0);
            if (token_offset < num_q && local_head < num_heads) {
                const uint16_t* row = p.q + ((uint64_t)(flat_begin + token_offset) * p.num_q_heads + first_q_head + local_head) * D;
                value = *reinterpret_cast<const uint4*>(row + chunk * 8);
            }
            *reinterpret_cast<uint4*>(q_lds + c * Smem::kQRowBytes + chunk * 16) = value;
        }
        __syncthreads();
    }

    // ---- tile schedule ---------------------------------------------------------------------
    const uint32_t tile_first = blk_lo >> 4;
    const uint32_t num_tiles = blk_hi > blk_lo ? ((blk_hi - 1) >> 4) - tile_first + 1 : 0;
    const uint32_t num_wave_tiles = num_tiles > (uint32_t)wave ? (num_tiles - wave + NWAVES - 1) / NWAVES : 0;

    const uint32_t* table = p.page_ids + ((uint64_t)req_slot * p.num_gqa_layers + layer) * p.pages_per_request_layer;
    const uint32_t tpp = p.tokens_per_page;
    const uint32_t tpp_shift = p.tokens_per_page_shift;
    const uint64_t kv_head_row0_k = ((uint64_t)kv_head * tpp) * ROW_BYTES;
    const uint64_t kv_head_row0_v = ((uint64_t)(p.num_kv_heads + kv_head) * tpp) * ROW_BYTES;

    // Page ids of 64 consecutive wave tiles per register; two registers alternate.
    uint32_t ids_a[2] = {0, 0}, ids_b[2] = {0, 0};
    auto load_ids = [&](uint32_t chunk, uint32_t (&ids)[2]) {
        const uint32_t j = chunk * 64 + lane;
        if (j < num_wave_tiles) {
            const uint32_t token = (tile_first + wave + NWAVES * j) << 4;
            const uint32_t last_page = p.pages_per_request_layer - 1;
            const uint32_t page0 = token >> tpp_shift;
            const uint32_t page1 = (token + 8) >> tpp_shift;
            ids[0] = table[page0 < last_page ? page0 : last_page];
            ids[1] = table[page1 < last_page ? page1 : last_page];
        }
    };
    load_ids(0, ids_a);
    if (num_wave_tiles > 64) load_ids(1, ids_b);

    auto load_tile = [&](uint32_t j, KvTile<D, KV8>& tile) {
        const uint32_t chunk = j >> 6;
        if ((j & 63) == 0 && chunk >= 1 && (chunk + 1) * 64 < num_wave_tiles) {
            if ((chunk + 1) & 1) load_ids(chunk + 1, ids_b); else load_ids(chunk + 1, ids_a);
        }
        const uint32_t sel0 = (chunk & 1) ? ids_b[0] : ids_a[0];
        const uint32_t sel1 = (chunk & 1) ? ids_b[1] : ids_a[1];
        uint32_t id0 = __builtin_amdgcn_readlane(sel0, j & 63);
        uint32_t id1 = __builtin_amdgcn_readlane(sel1, j & 63);
        const uint32_t first_token = (tile_first + wave + NWAVES * j) << 4;
        if (tpp == 8) {
            // A tile spans two 8-token pages; the half outside the block's KV range may have no
            // page assigned (its table entry can hold anything), so it borrows the other half's page.
            // Its K rows are masked and its V rows zeroed below.
            if (first_token + 8 >= blk_hi) id1 = id0;
            if (first_token + 8 <= blk_lo) id0 = id1;
        }
        tile.first_token = first_token;
        {
            const uint32_t row = r16;
            const uint32_t in_page = (first_token + row) & (tpp - 1);
            const uint64_t page = (row >= 8 ? id1 : id0);
            const unsigned char* base = p.kv_pages + page * p.page_bytes + kv_head_row0_k + (uint64_t)in_page * ROW_BYTES + g * 16;
#pragma unroll
            for (int i = 0; i < LOADS; ++i) tile.k[i] = load_streaming(base + i * 64);   // this block is the only reader
        }
        {
            const uint32_t row_in_load = lane / LANES_PER_ROW;
            const uint32_t chunk_in_row = lane % LANES_PER_ROW;
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const uint32_t row = i * ROWS_PER_LOAD + row_in_load;
                const uint32_t in_page = (first_token + row) & (tpp - 1);
                const uint64_t page = (row >= 8 ? id1 : id0);
                const unsigned char* source = p.kv_pages + page * p.page_bytes + kv_head_row0_v + (uint64_t)in_page * ROW_BYTES + chunk_in_row * 16;
                tile.v[i] = load_streaming(source);
            }
        }
    };

    // ---- online-softmax state --------------------------------------------------------------
    f32x4 acc[NT][MT];
    // Weights are exp2(score - ref) for a per-column reference that only moves when a score exceeds it by more than
    // kRescaleThreshold (so weights stay below 2^8 and the accumulator is rescaled a few times per block, not per
    // tile); lane_top is the lane's own largest score relative to ref, run_sum the lane's own part of the column sum.
    constexpr float kRescaleThreshold = 8.0f;
    float ref[NT], lane_top[NT], run_sum[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        ref[nt] = 0.0f;
        lane_top[nt] = -INFINITY;
        run_sum[nt] = 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    unsigned char* v_lds = v_lds_all + wave * 16 * Smem::kVRowBytes;
    const unsigned char* v_transposed = v_lds + (g * 4 + (r16 >> 2)) * Smem::kVRowBytes + (r16 & 3) * 8;

    auto compute_tile = [&](const KvTile<D, KV8>& tile) {
        const uint32_t first_token = tile.first_token;
        // S^T = K . Q^T
        f32x4 s[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) s[nt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 k_bits;
            if constexpr (KV8) {
                const uint4 codes = tile.k[ks >> 1];
                k_bits = fp8x8_to_bf16x8((ks & 1) ? make_uint2(codes.z, codes.w) : make_uint2(codes.x, codes.y));
            } else {
                k_bits = tile.k[ks];
            }
            const bf16x8 a = __builtin_bit_cast(bf16x8, k_bits);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                uint4 b_bits;
                if constexpr (kQInRegs) {
                    b_bits = q_frag[ks];
                } else {
                    b_bits = *reinterpret_cast<const uint4*>(q_lds + (nt * 16 + r16) * Smem::kQRowBytes + q_dim(ks, g) * 2);
                }
                s[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, b_bits), s[nt], 0, 0, 0);
            }
        }
        const bool interior = first_token >= all_lo && first_token + 16 <= all_hi;
        // Softmax weights go into the second MFMA as hi + lo bf16 pairs (p = hi + lo to ~2^-17): this kernel is
        // bandwidth-bound, so the second product is free and the weights keep f32-like accuracy as in the reference.
        uint32_t p_bits[NT][2], p_low[NT][2];
        float v[NT][4], tile_top[NT];
        bool lane_wants_move = false;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[nt][i] = __builtin_fmaf(s[nt][i], p.scale_log2e, -ref[nt]);
            if (!interior) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t token = first_token + g * 4 + i;
                    v[nt][i] = (token >= col_lo[nt] && token < col_hi[nt]) ? v[nt][i] : -INFINITY;
                }
            }
            tile_top[nt] = fmaxf(fmaxf(v[nt][0], v[nt][1]), fmaxf(v[nt][2], v[nt][3]));
            // a lane that has not seen a visible key yet cannot know whether its column has a reference
            lane_wants_move = lane_wants_move | (tile_top[nt] > kRescaleThreshold) | (lane_top[nt] == -INFINITY);
        }
        if (__builtin_amdgcn_ballot_w64(lane_wants_move) != 0) {
            // rare: the four lanes of a column agree on its maximum, move the reference, rescale what was accumulated
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float column_top = max_over_rows(tile_top[nt]);
                const float column_seen = max_over_rows(lane_top[nt]);
                const bool first = column_seen == -INFINITY;
                const bool move = column_top > kRescaleThreshold || (first && column_top > -INFINITY);
                const float shift = move ? column_top : 0.0f;
                const float alpha = first ? 0.0f : fast_exp2(-shift);   // nothing is accumulated before the first key
                ref[nt] += shift;
                lane_top[nt] -= shift;
                tile_top[nt] -= shift;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[nt][i] -= shift;
                run_sum[nt] *= alpha;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    asm volatile("" : "+a"(acc[nt][mt]));   // the move out of the AGPRs belongs to this branch
                    acc[nt][mt] *= alpha;
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            lane_top[nt] = fmaxf(lane_top[nt], tile_top[nt]);
            float e[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) e[i] = fast_exp2(v[nt][i]);
            run_sum[nt] += (e[0] + e[1]) + (e[2] + e[3]);
            p_bits[nt][0] = pack_bf16x2(e[0], e[1]);
            p_bits[nt][1] = pack_bf16x2(e[2], e[3]);
            p_low[nt][0] = pack_bf16x2(e[0] - bf16_bits_to_f32(p_bits[nt][0] & 0xffffu), e[1] - bf16_bits_to_f32(p_bits[nt][0] >> 16));
            p_low[nt][1] = pack_bf16x2(e[2] - bf16_bits_to_f32(p_bits[nt][1] & 0xffffu), e[3] - bf16_bits_to_f32(p_bits[nt][1] >> 16));
        }
        // V tile -> wave-private LDS (rows outside the block's KV range are zeroed: an unused
        // page slot may hold anything, and 0 * NaN would poison the accumulator).
        {
            const uint32_t row_in_load = lane / LANES_PER_ROW;
            const uint32_t chunk_in_row = lane % LANES_PER_ROW;
            const bool edge = first_token < blk_lo || first_token + 16 > blk_hi;
            auto stage = [&](int i, uint4 value) __attribute__((always_inline)) {
                const uint32_t row = i * ROWS_PER_LOAD + row_in_load;
                if constexpr (KV8) {
                    // sixteen codes -> sixteen bf16: the staged tile is bf16 whatever the page format
                    const uint4 low = fp8x8_to_bf16x8(make_uint2(value.x, value.y));
                    const uint4 high = fp8x8_to_bf16x8(make_uint2(value.z, value.w));
                    uint4* target = reinterpret_cast<uint4*>(v_lds + row * Smem::kVRowBytes + chunk_in_row * 32);
                    target[0] = low;
                    target[1] = high;
                } else {
                    *reinterpret_cast<uint4*>(v_lds + row * Smem::kVRowBytes + chunk_in_row * 16) = value;
                }
            };
            if (!edge) {
#pragma unroll
                for (int i = 0; i < LOADS; ++i) stage(i, tile.v[i]);
            } else {
#pragma unroll
                for (int i = 0; i < LOADS; ++i) {
                    const uint32_t token = first_token + i * ROWS_PER_LOAD + row_in_load;
                    stage(i, (token < blk_lo || token >= blk_hi) ? make_uint4(0, 0, 0, 0) : tile.v[i]);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // O^T += V^T . P^T
        // ds_read_b64_tr_b16: the lane passes (row 4g + r/4, dims mt*16 + 4*(r%4) .. +3) and receives dim mt*16 + r of
        // rows 4g .. 4g+3, which is the A fragment of V^T.
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const s16x4 a = __builtin_bit_cast(s16x4, lds_read_tr16(v_transposed + mt * 32));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint2 b_bits = make_uint2(p_bits[nt][0], p_bits[nt][1]);
                const uint2 b_low = make_uint2(p_low[nt][0], p_low[nt][1]);
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, __builtin_bit_cast(s16x4, b_bits), acc[nt][mt], 0, 0, 0);
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, __builtin_bit_cast(s16x4, b_low), acc[nt][mt], 0, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // The accumulator stays in the AGPR half of the register file from tile to tile (only the rare rescale moves
        // it through VGPRs); without the pin the compiler keeps a second copy in VGPRs and refreshes it after every tile.
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+a"(acc[nt][mt]));
    };

    // ---- main loop: a ring of register buffers, loads DEPTH tiles ahead ----------------------
    // Two tiles in flight per wave (8 KB each at D 128 on bf16 pages, half that on FP8 pages, where four in flight were
    // measured slower than two).  The ring is indexed with compile-time constants after unrolling.
    constexpr int DEPTH = kSlim ? 1 : kMapPrefetchDepth;
    if (num_wave_tiles > 0) {
        KvTile<D, KV8> ring[DEPTH + 1];
#pragma unroll
        for (int i = 0; i < DEPTH; ++i)
            if ((uint32_t)i < num_wave_tiles) load_tile(i, ring[i]);
        uint32_t j = 0;
        for (;;) {
            bool finished = false;
#pragma unroll
            for (int slot = 0; slot <= DEPTH; ++slot) {
                if (j + DEPTH < num_wave_tiles) load_tile(j + DEPTH, ring[(slot + DEPTH) % (DEPTH + 1)]);
                compute_tile(ring[slot]);
                if (++j >= num_wave_tiles) {
                    finished = true;
                    break;
                }
            }
            if (finished) break;
        }
    }

    // ---- merge the waves of the block ------------------------------------------------------
    float wave_ref[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        run_sum[nt] = sum_over_rows(run_sum[nt]);
        const float top = max_over_rows(lane_top[nt]);
        wave_ref[nt] = top == -INFINITY ? -INFINITY : ref[nt];     // a wave that saw no visible key has no reference
        if (g == 0) {
            float* stats = stats_lds + (wave * COLS + nt * 16 + r16) * 3;
            stats[0] = wave_ref[nt];
            stats[1] = run_sum[nt];
            stats[2] = top == -INFINITY ? -INFINITY : ref[nt] + top;   // the wave's true maximum
        }
    }
    __syncthreads();  // also: every wave is done with its V staging tile
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int c = nt * 16 + r16;
        float global_ref = -INFINITY, global_max = -INFINITY;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) {
            global_ref = fmaxf(global_ref, stats_lds[(w * COLS + c) * 3]);
            global_max = fmaxf(global_max, stats_lds[(w * COLS + c) * 3 + 2]);
        }
        float global_sum = 0.0f;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) {
            const float wave_sum = stats_lds[(w * COLS + c) * 3 + 1];
            if (wave_sum > 0.0f) global_sum += wave_sum * fast_exp2(stats_lds[(w * COLS + c) * 3] - global_ref);
        }
        const float own = (run_sum[nt] > 0.0f && global_sum > 0.0f) ? fast_exp2(wave_ref[nt] - global_ref) / global_sum : 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] *= own;
        if (wave == 0 && g == 0) {
            // published relative to the true maximum, as the partial-state contract says
            stats_lds[(NWAVES * COLS + c) * 3] = global_sum > 0.0f ? global_max * 0.6931471805599453f : -INFINITY;
            stats_lds[(NWAVES * COLS + c) * 3 + 1] = global_sum > 0.0f ? global_sum * fast_exp2(global_ref - global_max) : 0.0f;
        }
    }
    if constexpr (Smem::kTilePerWave) {
        // every wave stores its scaled accumulator into a tile of its own; the writer below adds the tiles up
        float* tile = o_lds + wave * (COLS * Smem::kORowFloats);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<f32x4*>(tile + r16 * Smem::kORowFloats + mt * 16 + g * 4) = acc[0][mt];
        __syncthreads();
    } else {
        for (int w = 0; w < NWAVES; ++w) {
            if (wave == w) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        float* cell = o_lds + (nt * 16 + r16) * Smem::kORowFloats + mt * 16 + g * 4;
                        f32x4 value = acc[nt][mt];
                        if (w > 0) value += *reinterpret_cast<const f32x4*>(cell);
                        *reinterpret_cast<f32x4*>(cell) = value;
                    }
                }
            }
            __syncthreads();
        }
    }

    // ---- write the block's partial state or final output ------------------------------------
    const uint32_t mode = p.output_mode;
    const bool fused = p.arrival_counters != nullptr && mode != kMapDirectBf16;
    for (int index = tid; index < COLS * (D / 4); index += NWAVES * 64) {
        const uint32_t c = index / (D / 4);
        const uint32_t d = (index - c * (D / 4)) * 4;
        const uint32_t token_offset = c / p.max_q_heads;
        const uint32_t local_head = c - token_offset * p.max_q_heads;
        if (token_offset >= num_q || local_head >= num_heads) continue;
        f32x4 value = *reinterpret_cast<const f32x4*>(o_lds + c * Smem::kORowFloats + d);
        if constexpr (Smem::kTilePerWave) {
#pragma unroll
            for (int w = 1; w < NWAVES; ++w) value += *reinterpret_cast<const f32x4*>(o_lds + (w * COLS + c) * Smem::kORowFloats + d);
        }
        const uint32_t q_head = first_q_head + local_head;
        uint64_t state;
        if (mode == kMapDirectBf16) {
            state = (uint64_t)(flat_begin + token_offset) * p.num_q_heads + q_head;
        } else {
            state = ((uint64_t)task * p.num_q_heads + q_head) * p.max_q_tokens + token_offset;
        }
        if (mode == kMapPartialF32) {
            float* target = reinterpret_cast<float*>(p.out) + state * D + d;
            if (fused) {
                coherent_store_u64(target, (uint64_t)__float_as_uint(value[0]) | ((uint64_t)__float_as_uint(value[1]) << 32));
                coherent_store_u64(target + 2, (uint64_t)__float_as_uint(value[2]) | ((uint64_t)__float_as_uint(value[3]) << 32));
            } else {
                *reinterpret_cast<f32x4*>(target) = value;
            }
        } else {
            if (mode == kMapDirectBf16 && p.gates != nullptr) value = gate_bf16x4(value, p.gates + state * D + d);
            const uint2 packed = make_uint2(pack_bf16x2(value[0], value[1]), pack_bf16x2(value[2], value[3]));
            uint16_t* target = reinterpret_cast<uint16_t*>(p.out) + state * D + d;
            if (fused) {
                coherent_store_u64(target, (uint64_t)packed.x | ((uint64_t)packed.y << 32));
            } else {
                *reinterpret_cast<uint2*>(target) = packed;
            }
        }
    }
    if (mode != kMapDirectBf16 && tid < COLS) {
        const uint32_t c = tid;
        const uint32_t token_offset = c / p.max_q_heads;
        const uint32_t local_head = c - token_offset * p.max_q_heads;
        if (token_offset < num_q && local_head < num_heads) {
            const uint64_t state = ((uint64_t)task * p.num_q_heads + first_q_head + local_head) * p.max_q_tokens + token_offset;
            if (fused) {
                coherent_store_f32(p.max_logits + state, stats_lds[(NWAVES * COLS + c) * 3]);
                coherent_store_f32(p.exp_sums + state, stats_lds[(NWAVES * COLS + c) * 3 + 1]);
            } else {
                p.max_logits[state] = stats_lds[(NWAVES * COLS + c) * 3];
                p.exp_sums[state] = stats_lds[(NWAVES * COLS + c) * 3 + 1];
            }
        }
    }

    // ---- fused Reduce: the last block of a (Q range, head group) merges all of its partial states ----------
    if (!fused) return;
    // Publishing the partial state to whichever block merges it.  Every store above is a device-coherent (sc1,
    // write-through) store: it is never held dirty in this XCD's L2, so what a release needs here is only that each wave
    // waits until its own stores have been acknowledged - the explicit wait below, which does not depend on what the
    // compiler puts in front of a barrier.  (A release fence at agent scope adds an L2 write-back per wave with nothing to
    // write back, and that alone takes a 2272-block launch from 114 to 209 us.)  The barrier then orders all waves' stores
    // before thread 0 signals arrival; the arrival is an acquire, so the block that sees the last one reads the others'
    // partial states - through device-coherent loads - after their stores.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t* flag_lds = reinterpret_cast<uint32_t*>(stats_lds);
    const uint32_t partial_begin = p.cu_partial_outputs[range_index];
    uint32_t partial_end = p.cu_partial_outputs[range_index + 1];
    if (partial_end > num_active_splits) partial_end = num_active_splits;
    if (tid == 0) {
        uint32_t* counter = p.arrival_counters + (uint64_t)range_index * gridDim.y + head_group_index;
        const uint32_t arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) + 1u;
        const uint32_t last = arrived == partial_end - partial_begin ? 1u : 0u;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // re-arm for the next launch
        flag_lds[0] = last;
    }
    __syncthreads();
    if (flag_lds[0] == 0u) return;
    {
        // Work units are (column, partial-slice) pairs; a group of D/4 lanes owns one unit at a time and walks
        // its partials with an online merge, eight partials' loads in flight at once.  With at least as many
        // columns as groups every column has one slice and a group writes its column's output directly;
        // with fewer columns the spare groups split the partial list and combine through LDS.
        constexpr int CHUNKS = D / 4;
        constexpr int GROUPS = NWAVES * 64 / CHUNKS;
        const int chunk = tid % CHUNKS;
        const uint32_t group = tid / CHUNKS;
        const uint32_t active_cols = num_q * p.max_q_heads;
        const uint32_t slices = active_cols >= (uint32_t)GROUPS ? 1u : (uint32_t)GROUPS / active_cols;
        const uint32_t num_units = active_cols * slices;
        float* unit_acc = o_lds;                 // [GROUPS][D]
        float* unit_stats = o_lds + GROUPS * D;  // [GROUPS][2]
        const bool f32_partials = mode == kMapPartialF32;
        for (uint32_t base = 0; base < num_units; base += GROUPS) {
            const uint32_t unit = base + group;
            const bool has_unit = unit < num_units;
            const uint32_t c = has_unit ? unit / slices : 0u;
            const uint32_t slice = unit - c * slices;
            const uint32_t token_offset = c / p.max_q_heads;
            const uint32_t local_head = c - token_offset * p.max_q_heads;
            const bool live = has_unit && local_head < num_heads;
            const uint32_t q_head = first_q_head + (live ? local_head : 0u);
            MergeState state = merge_state_empty();
            if (live) {
                merge_partial_slice<D, true>(state, p.max_logits, p.exp_sums, p.out, f32_partials, partial_begin + slice, partial_end, slices,
                                             partial_begin, p.num_q_heads, q_head, p.max_q_tokens, token_offset, chunk);
            }
            if (slices > 1u) {
                if (chunk == 0) {
                    unit_stats[group * 2] = state.run_max;
                    unit_stats[group * 2 + 1] = state.run_sum;
                }
                *reinterpret_cast<f32x4*>(unit_acc + group * D + chunk * 4) = state.acc;
                __syncthreads();
                if (live && slice == 0u) state = merge_combine_slices<D>(unit_stats, unit_acc, group, slices, chunk);
            }
            if (live && slice == 0u) {
                const uint64_t out_index = ((uint64_t)(flat_begin + token_offset) * p.num_q_heads + q_head) * D + chunk * 4;
                merge_store_output(state, p.final_output, p.gates, out_index);
            }
            if (slices > 1u) __syncthreads();
        }
    }
}

}  // namespace khm
