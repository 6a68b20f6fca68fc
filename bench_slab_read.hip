// Measurement aid of bench.py, not part of the attention library (it is built into a library of its own, beside
// bench.py): a kernel that only reads a list of 4 KB (or 2 KB) slabs of a K/V pool, in the lane layout and with the two tiles in
// flight per wave that the split-KV Map kernel uses, from a resident grid whose waves all get the same number of slabs.
// It does no arithmetic worth the name, has no dependent metadata loads, no merge and no imbalance, so its time for N
// bytes is what this memory system gives a launch of that size and access pattern; the benchmark reports it beside the
// Map kernel's time for the same bytes.  With `run_slabs` > 1 the list names runs of that many consecutive slabs
// (8 .. 64 KB contiguous, what a block covering several KV heads of a page would read), taken by neighbouring waves.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

// A slab is what one (page, plane, KV head) holds: 16 token rows, 4 KB at head_dim 128 on bf16 pages, 2 KB on FP8 pages.
// Each wave keeps 8 KB in flight: two slabs of 4 KB or four of 2 KB.
template <uint32_t SLAB>
__global__ __launch_bounds__(256) void calibration_slab_read_kernel(const unsigned char* pool, const uint32_t* slab_ids, uint32_t num_slabs,
                                                                     uint32_t run_shift, uint32_t* sink) {
    constexpr int LOADS = SLAB / 1024;       // 16-byte loads per lane and slab
    constexpr int FLIGHT = 8192 / SLAB;      // slabs requested before the first is consumed
    constexpr uint32_t ROW = SLAB / 16;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const uint32_t num_waves = gridDim.x * (blockDim.x >> 6);
    const uint32_t row = lane & 15, group = lane >> 4;
    uint32_t folded = 0;
    uint4 tile[FLIGHT][LOADS];
    auto request = [&](uint32_t slab, uint4 (&target)[LOADS]) {
        const uint64_t first = ((uint64_t)slab_ids[slab >> run_shift] << run_shift) + (slab & ((1u << run_shift) - 1u));
        const unsigned char* base = pool + first * SLAB + row * ROW + group * 16;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {   // streaming (nt) loads, as the Map kernels issue for bytes nobody reads twice
            typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
            const U32x4 v = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(base + i * 64));
            target[i] = make_uint4(v[0], v[1], v[2], v[3]);
        }
    };
    auto fold = [&](const uint4 (&source)[LOADS]) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) folded += source[i].x ^ source[i].y ^ source[i].z ^ source[i].w;
    };
    // groups of FLIGHT slabs: all requested, then all consumed
    uint32_t slab = wave;
    for (; slab + (FLIGHT - 1) * num_waves < num_slabs; slab += FLIGHT * num_waves) {
#pragma unroll
        for (int f = 0; f < FLIGHT; ++f) request(slab + f * num_waves, tile[f]);
#pragma unroll
        for (int f = 0; f < FLIGHT; ++f) fold(tile[f]);
    }
    for (; slab < num_slabs; slab += num_waves) {
        request(slab, tile[0]);
        fold(tile[0]);
    }
    if (folded == 0x9e3779b9u) sink[0] = folded;   // keeps the loads alive; practically never taken
}

}  // namespace

// Returns 0, or 1 for a bad argument, 2 for a HIP error (the launch is enqueued on `stream`, never synchronized).
extern "C" int bench_slab_read(const void* pool, uint64_t pool_bytes, const uint32_t* slab_ids, uint64_t slab_ids_bytes, uint32_t num_slabs,
                               uint32_t run_slabs, uint32_t slab_bytes, uint32_t blocks_per_cu, uint32_t* sink, uint64_t sink_bytes,
                               void* stream) {
    if (pool == nullptr || slab_ids == nullptr || sink == nullptr) return 1;
    if (run_slabs == 0 || (run_slabs & (run_slabs - 1)) != 0 || run_slabs > 64 || num_slabs % run_slabs != 0) return 1;
    if (num_slabs == 0 || (uint64_t)(num_slabs / run_slabs) * 4 > slab_ids_bytes) return 1;
    uint32_t run_shift = 0;
    while ((1u << run_shift) < run_slabs) ++run_shift;
    if (sink_bytes < 4 || blocks_per_cu < 1 || blocks_per_cu > 8) return 1;
    if (slab_bytes != 2048 && slab_bytes != 4096) return 1;
    if (pool_bytes < slab_bytes || pool_bytes / slab_bytes > 0xffffffffull) return 1;
    int device = 0, compute_units = 0;
    hipError_t status = hipGetDevice(&device);
    if (status == hipSuccess) status = hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device);
    if (status != hipSuccess || compute_units <= 0) return 2;
    // The slab ids are the caller's and are not read back here: ids beyond the pool are the caller's bug.
    auto kernel = slab_bytes == 2048 ? calibration_slab_read_kernel<2048> : calibration_slab_read_kernel<4096>;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)compute_units * blocks_per_cu), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const unsigned char*>(pool), slab_ids, num_slabs, run_shift, sink);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
