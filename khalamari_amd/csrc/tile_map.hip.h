// Tiled Map kernel for chunked prefill and wide verify blocks on gfx950 (bf16 MFMA, LDS-shared K/V tiles).
//
// Replaces gqa_sdpa_sliced_q_map / gqa_sdpa_sliced_q_per_head_map for Q tiles above 64 coordinates
// (crates/inference-backend-metal/src/components/metal/gqa_sdpa_sliced_q_map.metal:29-284,
// gqa_sdpa_sliced_q_per_head_map.metal:25-298): same task ABI (one block per map task template x KV head x
// Q-head range), same per-token visible range mask, same partial-state contract, and the direct-output mode.
//
// Work shape.  A block owns up to NWAVES * NTW * 16 (q_token, q_head) columns; each wave owns NTW 16-column
// tiles for the whole KV range, so there is no cross-wave merge.  KV is walked in BK-token tiles that all
// waves share through LDS, 32 tokens (one "slice") at a time:
//     S^T[32][cols] = K . Q^T        v_mfma_f32_16x16x32_bf16, K rows (ds_read_b128) as the A operand, Q in registers
//     online softmax per column      exp2 domain; the accumulator is rescaled only when a column's maximum moved far
//     O^T[D][cols] += V^T . P^T      v_mfma_f32_16x16x32_bf16; the V^T operand comes from row-major V in LDS through
//                                    ds_read_b64_tr_b16 (each lane receives 4 tokens of one dim), P stays in registers
// Memory.  K/V tiles go from HBM/L2 straight into LDS (global_load_lds_dwordx4, 1 KB per wave instruction) without
// passing through registers; NSTAGES tiles are in flight and one barrier per tile publishes them.  A direct load
// writes 64 consecutive 16-byte chunks, so rows cannot be padded; instead each lane fetches the chunk whose index is
// XOR-swizzled with the row, which makes both the b128 K reads and the transposed V reads bank-conflict free.
// Blocks are renumbered so that each XCD walks a contiguous run of the (KV head, template) list: the Q ranges of
// one sequence share their K/V through that XCD's L2 instead of each pulling it from HBM.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "device_math.hip.h"
#include "device_params.h"
#include "fp8_device.hip.h"

namespace khm {

// LDS tiles.  A tile is made of units: the 1024 bytes one wave load (64 lanes x 16 bytes) delivers, which the loading
// lanes may fill with any 64 of the 16-byte chunks of the rows the unit covers.
// LINEAR (bf16 pages): every fragment a lane reads during a slice sits at a fixed distance from the lane's first one,
// so the reads of a slice share one address register and differ in their immediate offsets only.  A unit covers 256
// bytes (128 dims) of four rows - at head dim 256 a row group has two units, one per half of the row - in pieces of 64
// bytes: piece q of row r at 256 q + 64 r, which keeps four neighbouring lanes of a wave load on 64 contiguous bytes
// of a page.  What keeps the lanes that the LDS serves in one pass on different banks: a ds_read_b128 is served in
// four passes of four lane quads each - quads {0,3,5,6}, {1,2,4,7}, {8,11,13,14}, {9,10,12,15} (measured: a layout
// that is conflict-free for sixteen consecutive lanes only shows one conflict cycle per pass) - so the four chunks of
// a K piece are permuted by (-chunk ^ row group) & 3; a ds_read_b64_tr_b16 is served in two passes of 32 lanes, which
// touch two V units, and V units lie 1056 bytes apart so that these fall on different halves of every 64 bytes.
// Other tiles (FP8 pages) keep rows whole and XOR the chunk index with the row (see the swizzles in the kernel).
template <int D, int BK, int NSTAGES, int ROW_BYTES = D * 2, bool LINEAR = false>
struct TileSmem {
    static_assert(!LINEAR || ROW_BYTES == 2 * D, "the linear layout is written for bf16 rows");
    static constexpr int kRowBytes = ROW_BYTES;
    static constexpr int kUnitsPerTile = BK * ROW_BYTES / 1024;
    static constexpr int kVUnitPitch = LINEAR ? 1056 : 1024;
    static constexpr int kKTileBytes = kUnitsPerTile * 1024;
    static constexpr int kVTileBytes = kUnitsPerTile * kVUnitPitch;
    static constexpr int kBytes = NSTAGES * (kKTileBytes + kVTileBytes);
};
// which kernels use the linear layout (the host sizes the dynamic LDS with the same rule)
constexpr bool tile_layout_is_linear(int head_dim, bool fp8_pages) { return (head_dim == 128 || head_dim == 256) && !fp8_pages; }


// 16 bytes per lane from global memory to LDS: lane l of the wave reads uniform_base + lane_offset and lands at
// lds_address + 16 * l (lds_address is wave-uniform and travels in M0).  Written as inline assembly on purpose: the
// compiler makes every LDS read wait for all direct-to-LDS loads it knows of (it cannot tell which tile a read
// touches), which would allow only one tile in flight; here the waits are explicit (wait_vmem_outstanding).
// STREAMING marks bytes that no other block of the launch reads again (the nt bit: a hint not to keep them cached).
template <bool STREAMING>
__device__ __forceinline__ void load_to_lds_b128(const unsigned char* uniform_base, uint32_t lane_offset, uint32_t lds_address) {
    if constexpr (STREAMING) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :
                     : "v"(lane_offset), "s"(uniform_base), "s"(lds_address)
                     : "memory", "m0");
    } else {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(lane_offset), "s"(uniform_base), "s"(lds_address)
                     : "memory", "m0");
    }
}

// Byte address of an LDS location as the hardware sees it.
__device__ __forceinline__ uint32_t lds_address_of(const unsigned char* pointer) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)pointer;
}

// Wait until at most COUNT of this wave's vector-memory operations are still in flight (they retire in order).
template <int COUNT>
__device__ __forceinline__ void wait_vmem_outstanding() {
    static_assert(COUNT >= 0 && COUNT < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COUNT) : "memory");
}

// Workgroup barrier for tiles that arrive through direct-to-LDS loads.  The caller has already waited (vmcnt) for
// the loads it needs, so only this wave's LDS reads must have completed; __syncthreads() carries a fence that
// would also drain every load still in flight and with it the whole multi-stage pipeline.
__device__ __forceinline__ void barrier_keeping_loads_in_flight() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// KV8: the pages hold FP8 E4M3FN codes, in one of two ways.
// Tiles with two column tiles per wave (MFMA-bound prefill) keep their LDS tiles bf16 in the same swizzled layout, so
// everything after the load is unchanged; the tile travels through registers (16 bytes = 16 codes per lane and load), is
// decoded there once and written to LDS one barrier before it is first read.  One tile is in flight in registers while
// two are consumed.
// Tiles with one column tile per wave (bandwidth-bound verify blocks) keep the raw codes in LDS: the tile goes from
// HBM/L2 straight into LDS like a bf16 one, half the bytes, and every wave decodes the fragments it reads (a K fragment
// is one ds_read_b64, a V^T fragment one ds_read_b64_tr_b8, four conversions each).  That repeats the decode in each of
// the four waves, which these tiles have the VALU time for, and takes the chain load -> registers -> decode -> LDS ->
// barrier off the critical path of a tile.
// DIRECT: the instantiation only ever writes final output (p.output_mode == kMapDirectBf16, which the host guarantees);
// it exists where following the largest score is worth compiling out, see the untracked slices below.
template <int D, int NTW, int NWAVES, int BK, int NSTAGES, int MIN_BLOCKS, bool KV8 = false, bool DIRECT = false>
__global__ __launch_bounds__(NWAVES * 64, MIN_BLOCKS) __attribute__((amdgpu_waves_per_eu(NWAVES * MIN_BLOCKS / 4, NWAVES * MIN_BLOCKS / 4)))
void tile_map_kernel(const MapParams p) {
    constexpr int KS = D / 32;                      // QK k-steps
    constexpr int MT = D / 16;                      // PV dim tiles
    constexpr int SL = BK / 32;                     // slices per tile
    constexpr int PAGE_ROW = D * (KV8 ? 1 : 2);     // bytes of one K/V row in a page
    constexpr int CPR = PAGE_ROW / 16;              // 16-byte chunks per K/V row in a page
    // The verify tiles (one column tile per wave, four waves: one block per KV range and KV head of a speculative block) are
    // the only readers of their K/V bytes, which therefore stream; the Q tiles of a prefill chunk share theirs through
    // the XCD's L2 (streaming loads there: 4.27 -> 4.40 ms).
    constexpr bool STREAM_KV = NTW == 1 && NWAVES == 4;
    constexpr bool LINEAR = tile_layout_is_linear(D, KV8);
    constexpr bool LINEAR_LOADS = LINEAR && !KV8;   // direct-to-LDS loads that fill the linear layout's units themselves
    constexpr int HALVES = LINEAR_LOADS ? D / 128 : 1;    // ... wave loads per row group (each takes 128 dims of four rows)
    constexpr int RPL = LINEAR_LOADS ? 4 : 64 / CPR;      // rows per wave load
    constexpr int UNITS = BK * CPR / 64;            // wave loads per plane and tile
    // PAIRED: the units divide evenly over the waves; a wave then loads K and V of the same units, which share their page
    // id and scalar base.  Otherwise (twelve waves over sixteen units) the 2 * UNITS loads of a tile are dealt out as one
    // list, two or three to a wave, and a wave with fewer repeats its last one so that every wave counts the same number
    // of loads per tile (the waits are compile-time constants).
    // FP8 tiles staged through registers have half as many units; when there are fewer than waves (twelve waves over
    // eight units) the first UNITS waves load one unit each and the others none (those loads are ordinary ones the
    // compiler waits for, so nothing has to be counted).
    constexpr int LOADERS = (KV8 && UNITS < NWAVES) ? UNITS : NWAVES;          // waves that load
    constexpr bool PAIRED = UNITS % LOADERS == 0;
    constexpr int UPW = PAIRED ? UNITS / LOADERS : 1;                          // units per loading wave (paired form)
    constexpr int LPW = PAIRED ? 2 * UPW : (2 * UNITS + NWAVES - 1) / NWAVES;  // loads per wave and tile
    constexpr int IDS = PAIRED ? UPW : LPW;                                    // page ids per wave and tile
    static_assert(PAIRED || !KV8, "FP8 tiles are written for evenly divided units");
    static_assert(LOADERS == NWAVES || (KV8 && !(NTW == 1 && NWAVES == 4)), "only register-staged FP8 tiles leave waves without loads");
    static_assert((SL == 1 || SL == 2) && NSTAGES >= 3 && NSTAGES <= 5, "unsupported tiling");
    constexpr bool RAW8 = KV8 && NTW == 1 && NWAVES == 4;   // raw FP8 codes in LDS, decoded by the waves that read them
    constexpr bool STAGED8 = KV8 && !RAW8;       // FP8 tiles decoded once on their way into bf16 LDS tiles
    static_assert(!STAGED8 || NSTAGES == 4, "the register-staged FP8 path is written for a ring of four tiles");
    using Smem = TileSmem<D, BK, NSTAGES, RAW8 ? D : 2 * D, LINEAR>;
    constexpr int ROW = Smem::kRowBytes;
    constexpr int V_UNIT = Smem::kVUnitPitch;
    // XOR swizzle of the 16-byte chunk position inside an LDS row, by tile row.  bf16 rows (and raw rows of 256 bytes)
    // alias bank for bank, so K reads spread sixteen rows over sixteen positions and the transposed V reads eight rows
    // over every second one; raw rows of 128 bytes alias in pairs and have eight chunks: both planes use (row / 2) % 8.
    auto k_swizzle_of = [](uint32_t row) -> uint32_t { return (RAW8 && D == 128) ? ((row >> 1) & 7u) : (row & 15u); };
    auto v_swizzle_of = [](uint32_t row) -> uint32_t { return RAW8 ? (D == 128 ? ((row >> 1) & 7u) : (row & 15u)) : ((row & 7u) << 1); };
    // Where chunk `chunk` (16 bytes) of tile row `row` sits inside its K or V tile in LDS.
    // Unit n of a tile (the n-th wave load of a plane): its first row, and its place among the tile's units in LDS.
    auto unit_first_row = [](uint32_t n) -> uint32_t { return (n / HALVES) * RPL; };
    auto unit_position = [](uint32_t n) -> uint32_t { return LINEAR_LOADS ? (n % HALVES) * (BK / 4) + n / HALVES : n; };
    auto k_place = [&](uint32_t row, uint32_t chunk) -> uint32_t {
        if constexpr (LINEAR) return ((chunk >> 4) * (BK / 4) + (row >> 2)) * 1024 + ((chunk >> 2) & 3u) * 256 + ((row & 3u) << 6) + ((((0u - chunk) ^ (row >> 2)) & 3u) << 4);
        else return row * ROW + ((chunk ^ k_swizzle_of(row)) << 4);
    };
    auto v_place = [&](uint32_t row, uint32_t chunk) -> uint32_t {
        if constexpr (LINEAR) return ((chunk >> 4) * (BK / 4) + (row >> 2)) * V_UNIT + ((chunk >> 2) & 3u) * 256 + ((row & 3u) << 6) + ((chunk & 3u) << 4);
        else return row * ROW + ((chunk ^ v_swizzle_of(row)) << 4);
    };
    // The inverse, for the lane that fills 16-byte slot `slot` of unit `unit` of a tile: row inside the tile and chunk.
    struct Source { uint32_t row, chunk; };
    auto k_source_of = [&](uint32_t unit, uint32_t slot) -> Source {
        if constexpr (LINEAR) return Source{unit_first_row(unit) + ((slot >> 2) & 3u), (unit % HALVES) * 16 + (slot >> 4) * 4 + ((0u - (slot ^ (unit / HALVES))) & 3u)};
        else { const uint32_t row = unit * RPL + slot / CPR; return Source{row, (slot % CPR) ^ k_swizzle_of(row)}; }
    };
    auto v_source_of = [&](uint32_t unit, uint32_t slot) -> Source {
        if constexpr (LINEAR) return Source{unit_first_row(unit) + ((slot >> 2) & 3u), (unit % HALVES) * 16 + (slot >> 4) * 4 + (slot & 3u)};
        else { const uint32_t row = unit * RPL + slot / CPR; return Source{row, (slot % CPR) ^ v_swizzle_of(row)}; }
    };

    extern __shared__ __align__(1024) unsigned char tile_smem[];
    unsigned char* k_lds = tile_smem;                                    // [NSTAGES][BK][ROW]
    unsigned char* v_lds = tile_smem + NSTAGES * Smem::kKTileBytes;      // [NSTAGES][units][V_UNIT]
    const uint32_t k_lds_address = lds_address_of(k_lds);
    const uint32_t v_lds_address = lds_address_of(v_lds);

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
    // Templates are taken last to first: within a request the later Q ranges see more keys, so the long blocks start
    // early and the short ones fill the end of the launch (2 % on a batch of 2048-token chunks).
    const uint32_t task = num_tasks - 1 - (uint32_t)(work % num_tasks);

    // ---- task decode (uniform) ---------------------------------------------------------------------------
    // every link of the chain arguments -> template -> Q range -> request slot is a scalar load, and what hangs on the
    // same link is requested together (see split_kv_map_kernel)
    fetch_all_arguments(p);
    const ReplayValues replay = resolve_replay_values(p);
    const uint32_t range_index = load_uniform_u32(p.templates, 3 * (uint64_t)task);
    const uint32_t kv_begin = load_uniform_u32(p.templates, 3 * (uint64_t)task + 1);
    const uint32_t kv_end = load_uniform_u32(p.templates, 3 * (uint64_t)task + 2);
    if (task >= replay.num_active_kv_splits) return;
    if (range_index >= replay.num_active_q_token_tiles) return;
    const uint32_t flat_begin = load_uniform_u32(p.q_token_ranges, 2 * (uint64_t)range_index);
    const uint32_t flat_end = load_uniform_u32(p.q_token_ranges, 2 * (uint64_t)range_index + 1);
    const uint32_t num_active_tokens = replay.num_active_tokens;
    if (flat_begin >= num_active_tokens || flat_end > num_active_tokens || flat_end <= flat_begin) return;
    uint32_t num_q = flat_end - flat_begin;
    if (num_q > p.max_q_tokens) num_q = p.max_q_tokens;
    const uint32_t req_slot = load_uniform_u32(p.req_slots, flat_begin);
    const uint32_t layer = replay.layer;

    const uint32_t head_range = head_group % p.num_q_head_ranges;
    const uint32_t kv_head = head_group / p.num_q_head_ranges;
    const uint32_t head_range_begin = head_range * p.max_q_heads;
    const uint32_t heads_left = p.q_heads_per_kv_head - head_range_begin;
    const uint32_t num_heads = heads_left < p.max_q_heads ? heads_left : p.max_q_heads;
    const uint32_t first_q_head = kv_head * p.q_heads_per_kv_head + head_range_begin;

    // ---- per-lane column facts ---------------------------------------------------------------------------
    auto column_token = [&](int nt) { return (uint32_t)((wave * NTW + nt) * 16 + r16) / p.max_q_heads; };
    auto column_head = [&](int nt) { return (uint32_t)((wave * NTW + nt) * 16 + r16) % p.max_q_heads; };
    uint32_t col_lo[NTW], col_hi[NTW];
    bool col_active[NTW];
    uint32_t blk_lo = 0xffffffffu, blk_hi = 0u, wave_all_lo = 0u, wave_all_hi = 0xffffffffu, min_span = 0xffffffffu;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        const uint32_t c = (wave * NTW + nt) * 16 + r16;
        const uint32_t token_offset = c / p.max_q_heads;
        const uint32_t local_head = c - token_offset * p.max_q_heads;
        col_active[nt] = token_offset < num_q && local_head < num_heads;
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
        // padding columns carry a zero Q row and are never stored, so they do not constrain anything
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
    // A wave none of whose columns is active (a request with fewer Q tokens than the tile has slots, fewer Q heads than
    // the tile has columns for) still loads its share of every K/V tile and meets every barrier, but computes nothing:
    // its LDS reads and matrix instructions would only take issue slots from the waves it shares a SIMD with.
    bool lane_has_column = false;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) lane_has_column = lane_has_column | col_active[nt];
    const bool wave_idle = __builtin_amdgcn_ballot_w64(lane_has_column) == 0;
    // a slice is "interior" for the wave when every active column of the wave sees all of its 32 tokens
    wave_all_lo = __builtin_amdgcn_readfirstlane(wave_all_lo);
    wave_all_hi = __builtin_amdgcn_readfirstlane(wave_all_hi);
    // block-wide KV range and shortest span: reduce the per-wave values through LDS
    uint32_t* range_lds = reinterpret_cast<uint32_t*>(tile_smem);
    if (lane == 0) {
        range_lds[wave * 3] = blk_lo;
        range_lds[wave * 3 + 1] = blk_hi;
        range_lds[wave * 3 + 2] = min_span;
    }
    __syncthreads();
    blk_lo = 0xffffffffu;
    blk_hi = 0u;
    min_span = 0xffffffffu;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) {
        const uint32_t lo = range_lds[w * 3], hi = range_lds[w * 3 + 1], span = range_lds[w * 3 + 2];
        blk_lo = lo < blk_lo ? lo : blk_lo;
        blk_hi = hi > blk_hi ? hi : blk_hi;
        min_span = span < min_span ? span : min_span;
    }
    blk_lo = __builtin_amdgcn_readfirstlane(blk_lo);
    blk_hi = __builtin_amdgcn_readfirstlane(blk_hi);
    // Rounding a softmax weight to bf16 costs up to 2^-9 of that weight; with few keys the weights are O(1) and
    // the error shows at the 1e-3 level.  Blocks with a column that sees at most kPreciseSpan keys therefore feed the
    // second MFMA with hi + lo bf16 pairs (the reference keeps P in f32); long contexts, where every weight is small,
    // use one.  On N(0,1) data a column over n keys has about n / e keys of comparable weight, so single rounding leaves
    // about 2^-9 / sqrt(3 n / e) of |v| in the output: 6e-4 at the worst of 4 million outputs with n just above 256
    // (1.05 % of an output of 0.05), half that from 1024 keys on.
    constexpr uint32_t kPreciseSpan = 1024;
    const bool precise = (uint32_t)__builtin_amdgcn_readfirstlane(min_span) <= kPreciseSpan;
    __syncthreads();   // range_lds is about to be overwritten by the first tile
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
            const uint16_t* row = p.q + ((uint64_t)(flat_begin + column_token(nt)) * p.num_q_heads + first_q_head + column_head(nt)) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) q_frag[nt][ks] = *reinterpret_cast<const uint4*>(row + ks * 32 + g * 8);
        }
    }

    // The Q loads have to be complete, in the compiler's eyes too, before the tile loop starts: a wait the compiler
    // placed inside the loop would also drain the direct-to-LDS loads in flight, of which it knows nothing.  The wait is
    // placed behind the requests of the first tiles (see below), so that both round trips to memory run side by side.
    auto settle_q_fragments = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
                U32x4 bits = __builtin_bit_cast(U32x4, q_frag[nt][ks]);
                asm volatile("" : "+v"(bits));
                q_frag[nt][ks] = __builtin_bit_cast(uint4, bits);
            }
    };

    // ---- tile schedule -------------------------------------------------------------------------------------
    const uint32_t first_group = blk_lo >> 4;                                   // 16-token groups
    const uint32_t num_groups = blk_hi > blk_lo ? ((blk_hi - 1) >> 4) - first_group + 1 : 0;
    const uint32_t num_slices = (num_groups + 1) / 2;
    const uint32_t num_tiles = (num_slices + SL - 1) / SL;
    const uint32_t first_token = first_group << 4;
    const uint32_t* table = p.page_ids + ((uint64_t)req_slot * p.num_gqa_layers + layer) * p.pages_per_request_layer;
    const uint32_t tpp = p.tokens_per_page;
    const uint32_t tpp_shift = p.tokens_per_page_shift;
    const uint64_t plane_k = ((uint64_t)kv_head * tpp) * PAGE_ROW;
    const uint64_t plane_v = ((uint64_t)(p.num_kv_heads + kv_head) * tpp) * PAGE_ROW;

    // A wave load covers RPL rows that lie inside one 8-token half of a 16-token group, before and after the clamp
    // below, so its page is wave-uniform: the page id travels through a scalar load, fetched one iteration before the
    // tile is issued, and the load address is a scalar base plus a 32-bit lane offset.
    // Rows outside [blk_lo, blk_hi) may hold anything (unused page slots): their loads are redirected to the nearest
    // visible token, so LDS only ever holds finite K/V and a zero weight really contributes zero.
    // Load j of this wave: which unit of the tile, K or V plane, and which of the wave's page ids it uses (all wave-uniform).
    const uint32_t first_load = PAIRED ? 0u : (uint32_t)(wave * 2 * UNITS) / NWAVES;
    const uint32_t num_loads = PAIRED ? (uint32_t)LPW : (uint32_t)((wave + 1) * 2 * UNITS) / NWAVES - first_load;
    auto load_index = [&](int j) -> uint32_t { return first_load + ((uint32_t)j < num_loads ? (uint32_t)j : num_loads - 1); };
    auto load_unit = [&](int j) -> uint32_t { return PAIRED ? (uint32_t)(wave * UPW + j / 2) : load_index(j) % UNITS; };
    auto load_is_v = [&](int j) -> bool { return PAIRED ? (j & 1) != 0 : load_index(j) >= (uint32_t)UNITS; };
    auto load_id = [](int j) -> int { return PAIRED ? j / 2 : j; };
    auto id_unit = [&](int i) -> uint32_t { return PAIRED ? (uint32_t)(wave * UPW + i) : load_unit(i); };
    auto load_lds_address = [&](int j, uint32_t stage) -> uint32_t {
        const uint32_t position = unit_position(load_unit(j));
        return load_is_v(j) ? v_lds_address + stage * Smem::kVTileBytes + position * V_UNIT : k_lds_address + stage * Smem::kKTileBytes + position * 1024;
    };
    auto load_source = [&](int j) -> Source { return load_is_v(j) ? v_source_of(load_unit(j), lane) : k_source_of(load_unit(j), lane); };

    typedef uint32_t TileIds __attribute__((ext_vector_type(IDS < 2 ? 2 : IDS)));
    auto fetch_ids = [&](uint32_t tile) __attribute__((always_inline)) -> TileIds {
        TileIds ids;
        const uint32_t last_page = p.pages_per_request_layer - 1;
#pragma unroll
        for (int i = 0; i < IDS; ++i) {
            uint32_t token = first_token + tile * BK + unit_first_row(id_unit(i));
            token = token < blk_lo ? blk_lo : token;
            token = token >= blk_hi ? blk_hi - 1 : token;
            const uint32_t page = token >> tpp_shift;
            ids[i] = load_uniform_u32(table, page < last_page ? page : last_page);
        }
        return ids;
    };
    // Lane offsets of a wave load inside its page.  A tile that lies wholly inside [blk_lo, blk_hi) needs no clamp and,
    // BK being a multiple of the page size, its offsets do not depend on the tile: those live in registers.  All loads
    // use one scalar base (the K plane of their page); the offsets of V loads carry the distance to the V plane.
    const uint32_t v_plane_distance = (uint32_t)(plane_v - plane_k);
    uint32_t lane_offset[LPW];
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const Source source = load_source(j);
        lane_offset[j] = ((first_token + source.row) & (tpp - 1)) * PAGE_ROW + (source.chunk << 4) + (load_is_v(j) ? v_plane_distance : 0u);
    }
    const unsigned char* const k_plane_base = p.kv_pages + plane_k;
    auto issue_tile = [&](uint32_t tile, const TileIds ids) __attribute__((always_inline)) {
        const uint32_t stage = tile % NSTAGES;
        const uint32_t tile_token = first_token + tile * BK;
        if (tile_token >= blk_lo && tile_token + BK <= blk_hi) {
#pragma unroll
            for (int j = 0; j < LPW; ++j)
                load_to_lds_b128<STREAM_KV>(k_plane_base + (uint64_t)ids[load_id(j)] * p.page_bytes, lane_offset[j], load_lds_address(j, stage));
            return;
        }
        // first or last tile of the range: rows outside it are redirected, which changes their offsets
#pragma unroll
        for (int j = 0; j < LPW; ++j) {
            const Source source = load_source(j);
            uint32_t token = tile_token + source.row;
            token = token < blk_lo ? blk_lo : token;
            token = token >= blk_hi ? blk_hi - 1 : token;
            const uint32_t offset = (token & (tpp - 1)) * PAGE_ROW + (source.chunk << 4) + (load_is_v(j) ? v_plane_distance : 0u);
            load_to_lds_b128<STREAM_KV>(k_plane_base + (uint64_t)ids[load_id(j)] * p.page_bytes, offset, load_lds_address(j, stage));
        }
    };

    // The same two steps for a tile known to lie wholly inside [blk_lo, blk_hi), as the steady-state loop requests them:
    // no clamps, no branches.
    auto fetch_ids_interior = [&](uint32_t tile) __attribute__((always_inline)) -> TileIds {
        TileIds ids;
        const uint32_t last_page = p.pages_per_request_layer - 1;
#pragma unroll
        for (int i = 0; i < IDS; ++i) {
            const uint32_t page = (first_token + tile * BK + unit_first_row(id_unit(i))) >> tpp_shift;
            ids[i] = load_uniform_u32(table, page < last_page ? page : last_page);   // the tile after the last one requested is read, not used
        }
        return ids;
    };
    auto issue_interior_tile = [&](uint32_t stage, const TileIds ids) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < LPW; ++j)
            load_to_lds_b128<STREAM_KV>(k_plane_base + (uint64_t)ids[load_id(j)] * p.page_bytes, lane_offset[j], load_lds_address(j, stage));
    };

    // FP8 pages: one tile in registers, decoded into the bf16 LDS layout the direct loads would have produced
    // (source chunk c of a K row lands at position c ^ (row & 15), of a V row at c ^ 2 (row & 7)).
    uint4 raw_k[STAGED8 ? UPW : 1], raw_v[STAGED8 ? UPW : 1];
    const bool loads_raw_tiles = LOADERS == NWAVES || wave < LOADERS;   // wave-uniform
    auto load_raw_tile = [&](uint32_t tile, const TileIds ids) __attribute__((always_inline)) {
        if (!loads_raw_tiles) return;
        const uint32_t load_row = lane / CPR;
        const uint32_t load_pos = lane % CPR;
        const uint32_t tile_token = first_token + tile * BK;
#pragma unroll
        for (int i = 0; i < UPW; ++i) {
            uint32_t token = tile_token + (wave * UPW + i) * RPL + load_row;
            token = token < blk_lo ? blk_lo : token;
            token = token >= blk_hi ? blk_hi - 1 : token;
            const unsigned char* page = p.kv_pages + (uint64_t)ids[i] * p.page_bytes;
            const uint32_t offset = (token & (tpp - 1)) * PAGE_ROW + load_pos * 16;
            raw_k[i] = *reinterpret_cast<const uint4*>(page + plane_k + offset);
            raw_v[i] = *reinterpret_cast<const uint4*>(page + plane_v + offset);
        }
    };
    // the same for a tile wholly inside [blk_lo, blk_hi): no clamps, lane offsets that do not depend on the tile
    uint32_t raw_lane_offset[STAGED8 ? UPW : 1];
    if constexpr (STAGED8) {
#pragma unroll
        for (int i = 0; i < UPW; ++i)
            raw_lane_offset[i] = ((first_token + (wave * UPW + i) * RPL + lane / CPR) & (tpp - 1)) * PAGE_ROW + (lane % CPR) * 16;
    }
    auto load_raw_tile_interior = [&](const TileIds ids) __attribute__((always_inline)) {
        if (!loads_raw_tiles) return;
#pragma unroll
        for (int i = 0; i < UPW; ++i) {
            const unsigned char* page = k_plane_base + (uint64_t)ids[i] * p.page_bytes;
            raw_k[i] = *reinterpret_cast<const uint4*>(page + raw_lane_offset[i]);
            raw_v[i] = *reinterpret_cast<const uint4*>(page + (plane_v - plane_k) + raw_lane_offset[i]);
        }
    };
    auto write_raw_tile = [&](uint32_t tile) __attribute__((always_inline)) {
        if (!loads_raw_tiles) return;
        const uint32_t load_row = lane / CPR;
        const uint32_t load_pos = lane % CPR;
        unsigned char* k_stage = k_lds + (tile % NSTAGES) * Smem::kKTileBytes;
        unsigned char* v_stage = v_lds + (tile % NSTAGES) * Smem::kVTileBytes;
#pragma unroll
        for (int i = 0; i < UPW; ++i) {
            const uint32_t row = (wave * UPW + i) * RPL + load_row;
            const uint4 k_low = fp8x8_to_bf16x8(make_uint2(raw_k[i].x, raw_k[i].y)), k_high = fp8x8_to_bf16x8(make_uint2(raw_k[i].z, raw_k[i].w));
            const uint4 v_low = fp8x8_to_bf16x8(make_uint2(raw_v[i].x, raw_v[i].y)), v_high = fp8x8_to_bf16x8(make_uint2(raw_v[i].z, raw_v[i].w));
            *reinterpret_cast<uint4*>(k_stage + k_place(row, 2 * load_pos)) = k_low;
            *reinterpret_cast<uint4*>(k_stage + k_place(row, 2 * load_pos + 1)) = k_high;
            *reinterpret_cast<uint4*>(v_stage + v_place(row, 2 * load_pos)) = v_low;
            *reinterpret_cast<uint4*>(v_stage + v_place(row, 2 * load_pos + 1)) = v_high;
        }
    };

    // ---- LDS read addresses (per lane, relative to the slice) -------------------------------------------------------
    // K: lane (r16, g) reads row rt*16 + r16, source chunk ks*4 + g, stored at position chunk ^ r16.
    // Raw FP8 rows: the lane's eight codes of k-step ks are half of source chunk ks*2 + g/2, stored at that index XOR the
    // row's swizzle (row tiles are sixteen rows apart, which leaves the swizzle alone).
    uint32_t k_offset[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        if constexpr (RAW8) k_offset[ks] = r16 * ROW + ((((uint32_t)ks * 2 + (g >> 1)) ^ k_swizzle_of(r16)) << 4) + (g & 1) * 8;
        else k_offset[ks] = k_place(r16, ks * 4 + g);   // layouts with fixed distances: k_offset[0] + 256 * ks
    }
    // V: lane (g, r) passes row 4g + r/4 (+16 for the second half), dims mt*16 + 4*(r%4) .. +3, i.e. source chunk
    // 2*mt + (r%4)/2, stored at position chunk ^ 2*(row & 7).
    // Raw FP8 rows (ds_read_b64_tr_b8: lane r of a 16-lane group passes eight consecutive bytes; lane i receives byte i % 8
    // of the rows passed by lanes i/8, i/8 + 2, ... i/8 + 14): lanes 2j and 2j + 1 pass the two halves of the sixteen
    // dims of token (j < 4 ? 4g + j : 16 + 4g + j - 4), so lane r receives dim mt*16 + r of exactly the eight tokens whose
    // weights it holds, in their order.
    const uint32_t v_row = RAW8 ? ((r16 >> 1) < 4 ? g * 4 + (r16 >> 1) : 16 + g * 4 + (r16 >> 1) - 4) : g * 4 + (r16 >> 2);
    const uint32_t v_swizzle = RAW8 ? v_swizzle_of(v_row) : ((r16 & 3) >> 1) ^ ((v_row & 7) << 1);
    const uint32_t v_base = LINEAR ? v_place(v_row, (r16 & 3) >> 1) + (r16 & 1) * 8 : v_row * ROW + (r16 & 1) * 8;
    constexpr uint32_t kKSliceBytes = LINEAR ? 8 * 1024 : 32 * ROW;      // from a 32-token slice of a tile to the next
    constexpr uint32_t kVSliceBytes = LINEAR ? 8 * V_UNIT : 32 * ROW;
    constexpr uint32_t kSixteenRows = LINEAR ? 4 * V_UNIT : 16 * ROW;    // V rows 16 apart in a tile
    constexpr uint32_t kSixteenKRows = LINEAR ? 4 * 1024 : 16 * ROW;     // K rows 16 apart in a tile
    auto v_fragment = [&](const unsigned char* v_src, int mt) __attribute__((always_inline)) -> bf16x8 {
        if constexpr (RAW8) {
            typedef int CodeWords __attribute__((ext_vector_type(2)));
            const unsigned char* address = v_src + v_base + (((uint32_t)mt ^ v_swizzle) << 4);
            const CodeWords codes = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CodeWords __attribute__((address_space(3)))*)(address));
            return __builtin_bit_cast(bf16x8, fp8x8_to_bf16x8(make_uint2((uint32_t)codes[0], (uint32_t)codes[1])));
        } else {
            const unsigned char* address = v_src + v_base + (LINEAR ? (uint32_t)((mt >> 3) * (BK / 4) * V_UNIT + ((mt & 7) >> 1) * 256 + (mt & 1) * 32) : ((mt * 2) ^ v_swizzle) << 4);
            const uint2 lo = __builtin_bit_cast(uint2, lds_read_tr16(address));
            const uint2 hi = __builtin_bit_cast(uint2, lds_read_tr16(address + kSixteenRows));
            return __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
        }
    };

    // ---- online-softmax state ------------------------------------------------------------------------------
    // Everything is kept in the log2 domain relative to ref[nt], the exponent reference of the lane's column.  The
    // reference only moves when a score exceeds it by more than kRescaleThreshold (or when the column sees its first
    // visible key), so the accumulators are rescaled rarely, and - what matters more - the hot path needs no
    // cross-lane maximum at all: each lane checks its own eight scores and one ballot decides whether any column of
    // the wave has to move.  lane_top[nt] is the largest score this lane has seen, relative to ref[nt]; the true
    // column maximum for the partial-state ABI is reduced across lanes once, in the epilogue.
    constexpr float kRescaleThreshold = 8.0f;
    // Interior slices of a direct-output block: a lane whose eight weights add up to more than 2^8 has a score more than
    // 5 above the reference; the reference then moves for every column whose maximum is more than 4 above it.
    constexpr float kSumTrigger = 256.0f;
    constexpr float kUntrackedMove = 4.0f;
    f32x4 acc[NTW][MT];
    float run_sum[NTW];
    float ref[NTW], lane_top[NTW];
    bool unanchored = false;   // before an untracked run: this lane has a column tile without a visible key so far
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        ref[nt] = 0.0f;
        lane_top[nt] = -INFINITY;
        run_sum[nt] = 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    struct Scores {
        f32x4 s[2][NTW];
    };
    // S^T of one 32-token slice
    auto scores_of = [&](const unsigned char* k_src, Scores& out) __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) out.s[rt][nt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                bf16x8 a;
                if constexpr (RAW8) {
                    a = __builtin_bit_cast(bf16x8, fp8x8_to_bf16x8(*reinterpret_cast<const uint2*>(k_src + k_offset[ks] + rt * kSixteenKRows)));
                } else {
                    a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(k_src + k_offset[ks] + rt * kSixteenKRows));
                }
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt)
                    out.s[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, q_frag[nt][ks]), out.s[rt][nt], 0, 0, 0);
            }
        }
    };

    // One slice: softmax update of the pending S^T, then P.V.  The S^T of the following slice is computed first: its
    // MFMAs depend on nothing the softmax produces, so the matrix pipe works on them while the VALU does the
    // exponentials (a software pipeline of depth one inside every wave).
    auto process_slice = [&](auto precise_tag, auto masked_tag, auto untracked_tag, uint32_t slice_first, Scores& scores,
                             const unsigned char* k_this, const unsigned char* k_next, const unsigned char* v_src, auto&& behind_the_scores) __attribute__((always_inline)) {
        constexpr bool PRECISE = decltype(precise_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;
        // UNTRACKED: the largest score is not followed (direct output needs no partial state).  The weights are computed
        // straight away and the lane's sum of them, which the slice needs anyway, tells whether a score ran away from
        // the reference: one compare per column tile instead of a maximum over the lane's eight scores.
        constexpr bool UNTRACKED = decltype(untracked_tag)::value != 0;
        constexpr bool ANCHORED = decltype(untracked_tag)::value == 2;   // untracked, and every column has its reference
        static_assert(!UNTRACKED || (!PRECISE && !MASKED), "the untracked slice is the plain interior one");
        Scores next;
        scores_of(k_next, next);
        behind_the_scores();   // address arithmetic and load issue of a later tile, while the matrix pipe works on S^T
        uint32_t p_bits[NTW][4], p_low[PRECISE ? NTW : 1][4];
        f32x4 (&s)[2][NTW] = scores.s;
        if constexpr (UNTRACKED) {
            float slice_sum[NTW];
            auto weights = [&]() __attribute__((always_inline)) {
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) {
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt) {
                        float e[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) e[i] = fast_exp2(s[rt][nt][i]);
                        p_bits[nt][2 * rt] = pack_bf16x2(e[0], e[1]);
                        p_bits[nt][2 * rt + 1] = pack_bf16x2(e[2], e[3]);
                        const float half_sum = (e[0] + e[1]) + (e[2] + e[3]);
                        slice_sum[nt] = rt == 0 ? half_sum : slice_sum[nt] + half_sum;
                    }
                }
            };
            auto relative_scores = [&]() __attribute__((always_inline)) {
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) s[rt][nt][i] = __builtin_fmaf(s[rt][nt][i], p.scale_log2e, -ref[nt]);
            };
            relative_scores();
            weights();
            float largest_sum = slice_sum[0];
#pragma unroll
            for (int nt = 1; nt < NTW; ++nt) largest_sum = fmaxf(largest_sum, slice_sum[nt]);
            bool lane_wants_move = !(largest_sum <= kSumTrigger);
            if constexpr (!ANCHORED) lane_wants_move = lane_wants_move | unanchored;
            if (__builtin_amdgcn_ballot_w64(lane_wants_move) != 0) {
                // rare: some lane's weights add up to more than kSumTrigger (one of its scores is then more than
                // kUntrackedMove above the reference), or a column has no reference yet.  The scores are computed again
                // from the slice's keys, still in LDS, so that the common path need not keep them beyond the weights.
                scores_of(k_this, scores);
                relative_scores();
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) {
                    const float lane_slice_top = fmaxf(fmaxf(fmaxf(s[0][nt][0], s[0][nt][1]), fmaxf(s[0][nt][2], s[0][nt][3])),
                                                       fmaxf(fmaxf(s[1][nt][0], s[1][nt][1]), fmaxf(s[1][nt][2], s[1][nt][3])));
                    const float column_top = max_over_rows(lane_slice_top);
                    const bool first = max_over_rows(lane_top[nt]) == -INFINITY;
                    const bool move = column_top > kUntrackedMove || first;   // every key of an interior slice is visible
                    const float shift = move ? column_top : 0.0f;
                    const float alpha = first ? 0.0f : fast_exp2(-shift);
                    ref[nt] += shift;
                    lane_top[nt] = fmaxf(lane_top[nt], lane_slice_top) - shift;   // only its finiteness is used from here on
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) s[rt][nt][i] -= shift;
                    run_sum[nt] *= alpha;
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] *= alpha;
                }
                weights();
            }
            unanchored = false;
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) run_sum[nt] += slice_sum[nt];
        } else {
            // scores relative to the column reference, the lane's maximum, and whether any column must move
            float slice_top[NTW];
            bool lane_wants_move = false;
    #pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
    #pragma unroll
                for (int rt = 0; rt < 2; ++rt)
    #pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float value = __builtin_fmaf(s[rt][nt][i], p.scale_log2e, -ref[nt]);
                        if constexpr (MASKED) {
                            const uint32_t token = slice_first + rt * 16 + g * 4 + i;
                            value = (token >= col_lo[nt] && token < col_hi[nt]) ? value : -INFINITY;
                        }
                        s[rt][nt][i] = value;
                    }
                slice_top[nt] = fmaxf(fmaxf(fmaxf(s[0][nt][0], s[0][nt][1]), fmaxf(s[0][nt][2], s[0][nt][3])),
                                      fmaxf(fmaxf(s[1][nt][0], s[1][nt][1]), fmaxf(s[1][nt][2], s[1][nt][3])));
                // a lane that has not seen a visible key yet cannot know whether its column has a reference
                lane_wants_move = lane_wants_move | (slice_top[nt] > kRescaleThreshold) | (lane_top[nt] == -INFINITY);
            }
            if (__builtin_amdgcn_ballot_w64(lane_wants_move) != 0) {
                // rare: agree per column (its four lanes) on the maximum, move the reference and rescale what was accumulated
    #pragma unroll
                for (int nt = 0; nt < NTW; ++nt) {
                    const float column_top = max_over_rows(slice_top[nt]);
                    const float column_seen = max_over_rows(lane_top[nt]);
                    const bool first = column_seen == -INFINITY;
                    const bool move = column_top > kRescaleThreshold || (first && column_top > -INFINITY);
                    const float shift = move ? column_top : 0.0f;
                    const float alpha = first ? 0.0f : fast_exp2(-shift);   // nothing is accumulated before the first key
                    ref[nt] += shift;
                    lane_top[nt] -= shift;
                    slice_top[nt] -= shift;
    #pragma unroll
                    for (int rt = 0; rt < 2; ++rt)
    #pragma unroll
                        for (int i = 0; i < 4; ++i) s[rt][nt][i] -= shift;
                    run_sum[nt] *= alpha;
    #pragma unroll
                    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] *= alpha;
                }
            }
    #pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                lane_top[nt] = fmaxf(lane_top[nt], slice_top[nt]);
                float slice_sum = 0.0f;
    #pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    float e[4];
    #pragma unroll
                    for (int i = 0; i < 4; ++i) e[i] = fast_exp2(s[rt][nt][i]);
                    const float half_sum = (e[0] + e[1]) + (e[2] + e[3]);
                    slice_sum = rt == 0 ? half_sum : slice_sum + half_sum;
                    p_bits[nt][2 * rt] = pack_bf16x2(e[0], e[1]);
                    p_bits[nt][2 * rt + 1] = pack_bf16x2(e[2], e[3]);
                    if constexpr (PRECISE) {
                        p_low[nt][2 * rt] = pack_bf16x2(e[0] - bf16_bits_to_f32(p_bits[nt][2 * rt] & 0xffffu), e[1] - bf16_bits_to_f32(p_bits[nt][2 * rt] >> 16));
                        p_low[nt][2 * rt + 1] = pack_bf16x2(e[2] - bf16_bits_to_f32(p_bits[nt][2 * rt + 1] & 0xffffu), e[3] - bf16_bits_to_f32(p_bits[nt][2 * rt + 1] >> 16));
                    }
                }
                run_sum[nt] += slice_sum;
            }
        }
        // O^T += V^T . P^T over the 32 tokens: k = 8g + j <-> token (j < 4 ? 4g + j : 16 + 4g + j - 4) of the slice.
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const bf16x8 a = v_fragment(v_src, mt);
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                const uint4 b_bits = make_uint4(p_bits[nt][0], p_bits[nt][1], p_bits[nt][2], p_bits[nt][3]);
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, b_bits), acc[nt][mt], 0, 0, 0);
                if constexpr (PRECISE) {
                    const uint4 low_bits = make_uint4(p_low[nt][0], p_low[nt][1], p_low[nt][2], p_low[nt][3]);
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, low_bits), acc[nt][mt], 0, 0, 0);
                }
            }
        }
        scores = next;
    };
    // ---- main loop --------------------------------------------------------------------------------------------------
    // Tile j lives in stage j % NSTAGES.  Because a slice's S^T is computed one slice ahead, tile j + 1 has to be
    // readable while tile j is consumed: at the top of tile j the wave waits for its own loads of tile j + 1 and the
    // barrier publishes them; every wave has then left tile j-1, whose stage receives tile j + NSTAGES - 1.
    // The wave walks its tiles in three runs - masked head, interior, masked tail - so that every loop holds exactly one
    // variant of the slice code; all waves pass the same number of barriers whatever their split.
    auto wait_for_tile = [&](uint32_t tile) __attribute__((always_inline)) {
        // loads issued so far reach tile min(issued_until, num_tiles - 1); those after `tile` may stay in flight
        const uint32_t newer = num_tiles - 1 - tile < (uint32_t)(NSTAGES - 2) ? num_tiles - 1 - tile : (uint32_t)(NSTAGES - 2);
        if (NSTAGES >= 5 && newer >= 3) wait_vmem_outstanding<3 * LPW>();
        else if (NSTAGES >= 4 && newer >= 2) wait_vmem_outstanding<2 * LPW>();
        else if (newer >= 1) wait_vmem_outstanding<LPW>();
        else wait_vmem_outstanding<0>();
    };
    auto k_slice = [&](uint32_t slice) __attribute__((always_inline)) -> const unsigned char* {
        return k_lds + ((slice / SL) % NSTAGES) * Smem::kKTileBytes + (slice % SL) * kKSliceBytes;
    };
    auto v_slice = [&](uint32_t slice) __attribute__((always_inline)) -> const unsigned char* {
        return v_lds + ((slice / SL) % NSTAGES) * Smem::kVTileBytes + (slice % SL) * kVSliceBytes;
    };
    Scores pending;
    TileIds upcoming = fetch_ids(NSTAGES - 1);
    // FP8 pages: decode tile + 2 from registers into LDS, request tile + 3.  The MFMA-bound tiles (two column tiles per
    // wave) do it behind the first S^T of the tile like the bf16 path requests its loads (1.6 % on config 5); the
    // bandwidth-bound verify tiles do it straight after the barrier, where the decoded tile is ready soonest (2 %).
    constexpr bool kRawTileBehindScores = NTW >= 2;
    auto advance_raw_tiles = [&](uint32_t tile) __attribute__((always_inline)) {
        if (tile + 2 < num_tiles) write_raw_tile(tile + 2);
        if (tile + 3 < num_tiles) {
            load_raw_tile(tile + 3, upcoming);
            upcoming = fetch_ids(tile + 4);
        }
    };
    auto run_tiles = [&](auto precise_tag, auto masked_tag, auto untracked_tag, uint32_t tile_begin, uint32_t tile_end) __attribute__((always_inline)) {
        for (uint32_t tile = tile_begin; tile < tile_end; ++tile) {
            if constexpr (STAGED8) {
                // tile + 1 was written to LDS during the previous tile; tile + 2 sits in registers, tile + 3 is requested
                barrier_keeping_loads_in_flight();
                if constexpr (!kRawTileBehindScores) advance_raw_tiles(tile);
            } else {
                // at this point the loads of tiles up to tile + NSTAGES - 2 have been issued
                if (tile + 1 < num_tiles) {
                    const uint32_t last_issued = tile + NSTAGES - 2 < num_tiles - 1 ? tile + NSTAGES - 2 : num_tiles - 1;
                    const uint32_t newer = last_issued - (tile + 1);
                    if (NSTAGES >= 5 && newer >= 2) wait_vmem_outstanding<2 * LPW>();
                    else if (newer >= 1) wait_vmem_outstanding<LPW>();
                    else wait_vmem_outstanding<0>();
                }
                barrier_keeping_loads_in_flight();
            }
            // The stage of tile - 1 is free from the barrier on; its next tenant is requested behind the first S^T of
            // this tile rather than straight after the barrier, where all waves would do address arithmetic at once
            // with the matrix pipe idle.
            auto request_next = [&]() __attribute__((always_inline)) {
                if constexpr (!STAGED8) {
                    if (tile + NSTAGES - 1 < num_tiles) {
                        issue_tile(tile + NSTAGES - 1, upcoming);
                        upcoming = fetch_ids(tile + NSTAGES);
                    }
                }
                if constexpr (STAGED8 && kRawTileBehindScores) advance_raw_tiles(tile);
            };
            auto nothing = []() __attribute__((always_inline)) {};
#pragma unroll
            for (int k = 0; k < SL; ++k) {
                const uint32_t slice = tile * SL + k;
                if (k == 0 || slice < num_slices) {
                    const uint32_t following = slice + 1 < num_slices ? slice + 1 : slice;   // the last one recomputes itself, unused
                    if (k == 0) process_slice(precise_tag, masked_tag, untracked_tag, first_token + slice * 32, pending, k_slice(slice), k_slice(following), v_slice(slice), request_next);
                    else process_slice(precise_tag, masked_tag, untracked_tag, first_token + slice * 32, pending, k_slice(slice), k_slice(following), v_slice(slice), nothing);
                }
            }
        }
    };
    // Steady state of an interior run (direct loads; weights untracked with every column anchored, or tracked): every tile of
    // [tile_begin, tile_end) has its successor's first slice in the range, and the tile NSTAGES - 1 ahead exists and lies
    // wholly inside the block's KV range.  One straight-line body per tile: a fixed wait, the barrier, unconditional
    // requests; the compiler is free to mix the S^T of the next slice with the softmax of this one.
    auto run_steady_tiles = [&](auto untracked_anchored, uint32_t tile_begin, uint32_t tile_end) __attribute__((always_inline)) {
        constexpr std::false_type no{};
        TileIds ahead = fetch_ids_interior(tile_begin + NSTAGES - 1);
        for (uint32_t tile = tile_begin; tile < tile_end; ++tile) {
            // direct loads: tile + 1 has landed, tiles up to tile + NSTAGES - 2 are requested; FP8 tiles staged through
            // registers: tile + 1 is in LDS, tile + 2 in registers, tile + 3 is requested here (the compiler waits for it)
            if constexpr (!STAGED8) wait_vmem_outstanding<(NSTAGES - 3) * LPW>();
            barrier_keeping_loads_in_flight();
            const uint32_t stage = tile % NSTAGES, next_stage = (tile + 1) % NSTAGES, free_stage = (tile + NSTAGES - 1) % NSTAGES;
            const unsigned char* k_tile = k_lds + stage * Smem::kKTileBytes;
            const unsigned char* v_tile = v_lds + stage * Smem::kVTileBytes;
            auto request_next = [&]() __attribute__((always_inline)) {
                if constexpr (STAGED8) {
                    write_raw_tile(tile + 2);
                    load_raw_tile_interior(ahead);
                } else {
                    issue_interior_tile(free_stage, ahead);
                }
                ahead = fetch_ids_interior(tile + NSTAGES);
            };
            auto nothing = []() __attribute__((always_inline)) {};
            const unsigned char* k_following = k_lds + next_stage * Smem::kKTileBytes;
            if constexpr (SL == 2) {
                process_slice(no, no, untracked_anchored, 0u, pending, k_tile, k_tile + kKSliceBytes, v_tile, request_next);
                process_slice(no, no, untracked_anchored, 0u, pending, k_tile + kKSliceBytes, k_following, v_tile + kVSliceBytes, nothing);
            } else {
                process_slice(no, no, untracked_anchored, 0u, pending, k_tile, k_following, v_tile, request_next);
            }
        }
    };

    if (num_tiles > 0) {
        if constexpr (STAGED8) {
            // tiles 0 and 1 into LDS, tile 2 into registers
            load_raw_tile(0, fetch_ids(0));
            write_raw_tile(0);
            if (num_tiles > 1) {
                load_raw_tile(1, fetch_ids(1));
                write_raw_tile(1);
            }
            if (num_tiles > 2) load_raw_tile(2, fetch_ids(2));
            settle_q_fragments();
        } else {
#pragma unroll
            for (int t = 0; t < NSTAGES - 1; ++t)
                if ((uint32_t)t < num_tiles) issue_tile(t, fetch_ids(t));
            settle_q_fragments();
            // publish tile 0 and start the pipeline with the scores of the first slice
            wait_for_tile(0);
        }
        barrier_keeping_loads_in_flight();
        if (wave_idle) {
            // the loads, waits and barriers of run_tiles, nothing else
            for (uint32_t tile = 0; tile < num_tiles; ++tile) {
                if constexpr (STAGED8) {
                    barrier_keeping_loads_in_flight();
                    advance_raw_tiles(tile);
                } else {
                    if (tile + 1 < num_tiles) {
                        const uint32_t last_issued = tile + NSTAGES - 2 < num_tiles - 1 ? tile + NSTAGES - 2 : num_tiles - 1;
                        const uint32_t newer = last_issued - (tile + 1);
                        if (NSTAGES >= 5 && newer >= 2) wait_vmem_outstanding<2 * LPW>();
                        else if (newer >= 1) wait_vmem_outstanding<LPW>();
                        else wait_vmem_outstanding<0>();
                    }
                    barrier_keeping_loads_in_flight();
                    if (tile + NSTAGES - 1 < num_tiles) {
                        issue_tile(tile + NSTAGES - 1, upcoming);
                        upcoming = fetch_ids(tile + NSTAGES);
                    }
                }
            }
            return;   // no column of this wave is stored
        }
        scores_of(k_slice(0), pending);
        // tiles [0, head_end) and [tail_begin, num_tiles) hold tokens some active column of the wave does not see
        uint32_t head_end = wave_all_lo > first_token ? (wave_all_lo - first_token + BK - 1) / BK : 0;
        head_end = head_end < num_tiles ? head_end : num_tiles;
        uint32_t tail_begin = wave_all_hi > first_token ? (wave_all_hi - first_token) / BK : 0;
        tail_begin = tail_begin < num_tiles ? tail_begin : num_tiles;
        tail_begin = tail_begin > head_end ? tail_begin : head_end;
        constexpr std::true_type yes{};
        constexpr std::false_type no{};
        if (precise) {
            run_tiles(yes, yes, no, 0, head_end);
            run_tiles(yes, no, no, head_end, tail_begin);
            run_tiles(yes, yes, no, tail_begin, num_tiles);
        } else {
            run_tiles(no, yes, no, 0, head_end);
            // tiles t with t + NSTAGES - 1 a whole tile inside [blk_lo, blk_hi), (t + NSTAGES) * BK <= blk_hi - first_token, run in
            // the steady-state loop
            uint32_t steady_limit = head_end;
            {
                const uint32_t whole_tiles = (blk_hi - first_token) / BK;
                steady_limit = whole_tiles >= (uint32_t)NSTAGES ? whole_tiles - (NSTAGES - 1) : 0;
                steady_limit = steady_limit < tail_begin ? steady_limit : tail_begin;
                steady_limit = steady_limit > head_end ? steady_limit : head_end;
            }
            if constexpr (DIRECT) {
                // no partial state to hand on: the interior slices need not follow the largest score
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) unanchored = unanchored | (lane_top[nt] == -INFINITY);
                uint32_t steady_begin = head_end;
                if (steady_limit > head_end && __builtin_amdgcn_ballot_w64(unanchored) != 0) {
                    // a column without a reference yet: the general slice anchors it
                    run_tiles(no, no, yes, head_end, head_end + 1);
                    steady_begin = head_end + 1;
                }
                if (steady_limit > steady_begin) {
                    run_steady_tiles(std::integral_constant<int, 2>{}, steady_begin, steady_limit);
                    upcoming = fetch_ids(steady_limit + NSTAGES - 1);
                    steady_begin = steady_limit;
                }
                run_tiles(no, no, yes, steady_begin, tail_begin);
            } else {
                if (steady_limit > head_end) {
                    run_steady_tiles(no, head_end, steady_limit);
                    upcoming = fetch_ids(steady_limit + NSTAGES - 1);
                }
                run_tiles(no, no, no, steady_limit, tail_begin);
            }
            run_tiles(no, yes, no, tail_begin, num_tiles);
        }
    }

    // ---- epilogue: every wave owns its columns, no cross-wave merge ------------------------------------------------
    const uint32_t mode = DIRECT ? (uint32_t)kMapDirectBf16 : p.output_mode;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
        // the lanes of a column each hold the sum over their tokens, relative to ref[nt]
        float total = run_sum[nt];
        total = sum_over_rows(total);
        const float column_top = max_over_rows(lane_top[nt]);   // the column's largest score, relative to ref[nt]
        if (!col_active[nt]) continue;
        const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
        const uint32_t q_head = first_q_head + column_head(nt);
        uint64_t row;
        if (mode == kMapDirectBf16) {
            row = (uint64_t)(flat_begin + column_token(nt)) * p.num_q_heads + q_head;
        } else {
            row = ((uint64_t)task * p.num_q_heads + q_head) * p.max_q_tokens + column_token(nt);
            if (g == 0) {
                p.exp_sums[row] = total > 0.0f ? total * fast_exp2(-column_top) : 0.0f;
                p.max_logits[row] = total > 0.0f ? (ref[nt] + column_top) * 0.6931471805599453f : -INFINITY;
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            f32x4 value = acc[nt][mt] * inverse;
            const uint32_t d = mt * 16 + g * 4;
            // direct output of a gated layer: the sigmoid gate of the final bf16 value, as the Reduce applies it
            if (mode == kMapDirectBf16 && p.gates != nullptr) value = gate_bf16x4(value, p.gates + row * D + d);
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
