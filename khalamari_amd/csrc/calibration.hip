// Measurement aid, not part of the attention path: a kernel that only reads a list of 4 KB slabs of a K/V pool, in
// the lane layout and with the two tiles in flight per wave that the split-KV Map kernel uses, from a resident grid
// whose waves all get the same number of slabs.  It does no arithmetic worth the name, has no dependent metadata
// loads, no merge and no imbalance, so its time for N bytes is what this memory system gives a launch of that size
// and access pattern; the benchmark reports it beside the Map kernel's time for the same bytes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"

namespace khm {

constexpr uint32_t kSlabBytes = 4096;   // 16 token rows of one KV head at head_dim 128, bf16

__global__ __launch_bounds__(256) void calibration_slab_read_kernel(const unsigned char* pool, const uint32_t* slab_ids, uint32_t num_slabs,
                                                                     uint32_t* sink) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const uint32_t num_waves = gridDim.x * (blockDim.x >> 6);
    const uint32_t row = lane & 15, group = lane >> 4;
    uint32_t folded = 0;
    uint4 tile[2][4];
    auto request = [&](uint32_t slab, uint4 (&target)[4]) {
        const unsigned char* base = pool + (uint64_t)slab_ids[slab] * kSlabBytes + row * 256 + group * 16;
#pragma unroll
        for (int i = 0; i < 4; ++i) target[i] = *reinterpret_cast<const uint4*>(base + i * 64);
    };
    auto fold = [&](const uint4 (&source)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) folded += source[i].x ^ source[i].y ^ source[i].z ^ source[i].w;
    };
    // pairs of slabs: both requested, then both consumed
    uint32_t slab = wave;
    for (; slab + num_waves < num_slabs; slab += 2 * num_waves) {
        request(slab, tile[0]);
        request(slab + num_waves, tile[1]);
        fold(tile[0]);
        fold(tile[1]);
    }
    if (slab < num_slabs) {
        request(slab, tile[0]);
        fold(tile[0]);
    }
    if (folded == 0x9e3779b9u) sink[0] = folded;   // keeps the loads alive; practically never taken
}

}  // namespace khm

using namespace khm;

extern "C" int khm_calibration_slab_read(khm_buffer pool, khm_buffer slab_ids, uint32_t num_slabs, uint32_t blocks_per_cu, khm_buffer sink,
                                         void* stream) {
    clear_error();
    KHM_REQUIRE(pool.ptr != nullptr && slab_ids.ptr != nullptr && sink.ptr != nullptr, "pool, slab_ids and sink must not be null");
    KHM_REQUIRE(num_slabs > 0 && (uint64_t)num_slabs * 4 <= slab_ids.len_bytes, "slab_ids holds fewer than num_slabs entries");
    KHM_REQUIRE(sink.len_bytes >= 4, "sink needs four bytes");
    KHM_REQUIRE(blocks_per_cu >= 1 && blocks_per_cu <= 8, "blocks_per_cu must be 1..8");
    KHM_REQUIRE(pool.len_bytes >= kSlabBytes && pool.len_bytes / kSlabBytes <= 0xffffffffull, "pool must hold 1 .. 2^32-1 slabs of 4096 bytes");
    int device = 0, compute_units = 0;
    hipError_t status = hipGetDevice(&device);
    if (status == hipSuccess) status = hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device);
    if (status != hipSuccess || compute_units <= 0) return fail(KHM_ERR_HIP, "could not read the compute unit count: %s", hipGetErrorString(status));
    // The slab ids are the caller's and are not read back here: ids beyond the pool are the caller's bug, as with page ids.
    hipLaunchKernelGGL(calibration_slab_read_kernel, dim3((uint32_t)compute_units * blocks_per_cu), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const unsigned char*>(pool.ptr), static_cast<const uint32_t*>(slab_ids.ptr), num_slabs,
                       static_cast<uint32_t*>(sink.ptr));
    const hipError_t launched = hipGetLastError();
    if (launched != hipSuccess) return fail(KHM_ERR_HIP, "calibration slab read launch failed: %s", hipGetErrorString(launched));
    return KHM_OK;
}
