// Measurement aid of bench.py, not part of the attention library (built into libbench_slab_read.so beside bench.py).
//
// What rate do the matrix cores of this chip sustain when they do nothing but bf16 MFMA instructions back to back, and
// at which shader clock?  The published dense bf16 peak (2.5 PFLOP/s) is 256 CUs x 4 SIMDs x 1024 flop/clk at 2.4 GHz.
// A loop of MFMAs on operands that are all 1.0 reaches it: nothing toggles in the multipliers and the chip stays at
// its top clock.  With operands drawn from N(0, 1) - what attention on real Q, K, V looks like - the same loop draws
// enough power that the clock governor settles well below 2.4 GHz, and that lower product of clock and width is the
// ceiling for any kernel on real data, however well it feeds the matrix cores.  bench.py reports it beside the prefill
// roofline fraction, which is quoted against the published peak.
//
// One block of eight waves per CU (two per SIMD), four independent accumulators per wave, no memory traffic in the
// loop.  The clock is the ratio of the shader clock counter (s_memtime) to the constant 100 MHz counter
// (s_memrealtime) over the loop, read by wave 0 of block 0.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kThreads = 512;
constexpr uint32_t kOperandSets = 4;
constexpr uint32_t kFlopsPerStep = 8 * 32768;   // per wave and loop step, both tile shapes

// TILE32: v_mfma_f32_32x32x16_bf16 (8 per step), else v_mfma_f32_16x16x32_bf16 (16 per step)
template <bool TILE32>
__global__ __launch_bounds__(kThreads) void mfma_sustained_kernel(const uint4* operands, float* sink, uint64_t* counters, uint32_t steps) {
    bf16x8 a[kOperandSets], b[kOperandSets];
#pragma unroll
    for (uint32_t i = 0; i < kOperandSets; ++i) {
        a[i] = __builtin_bit_cast(bf16x8, operands[threadIdx.x + i * kThreads]);
        b[i] = __builtin_bit_cast(bf16x8, operands[threadIdx.x + (kOperandSets + i) * kThreads]);
    }
    f32x16 wide[4];
    f32x4 narrow[8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) wide[i][j] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) narrow[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const uint64_t clock_begin = __builtin_amdgcn_s_memtime(), real_begin = __builtin_amdgcn_s_memrealtime();
    for (uint32_t step = 0; step < steps; ++step) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (TILE32) {
                wide[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i & 3], b[(i >> 1) & 3], wide[i & 3], 0, 0, 0);
            } else {
                narrow[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 3], b[(i >> 1) & 3], narrow[i], 0, 0, 0);
                narrow[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(i + 1) & 3], b[(i >> 1) & 3], narrow[i], 0, 0, 0);
            }
        }
    }
    const uint64_t clock_end = __builtin_amdgcn_s_memtime(), real_end = __builtin_amdgcn_s_memrealtime();
    float folded = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) folded += wide[i][j];
#pragma unroll
    for (int i = 0; i < 8; ++i) folded += narrow[i][0] + narrow[i][1] + narrow[i][2] + narrow[i][3];
    sink[blockIdx.x * kThreads + threadIdx.x] = folded;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        counters[0] = clock_end - clock_begin;
        counters[1] = real_end - real_begin;
    }
}

// One wave that sleeps for `delay_ticks` of the 100 MHz counter, then reads both counters, sleeps for `window_ticks`
// and reads them again: launched on a second stream while another kernel runs, it reports the shader clock of the XCD
// it lands on while that kernel runs (an indication, not a chip-wide average).  The loops end on the real-time counter
// and on an iteration cap.
__global__ __launch_bounds__(64) void clock_probe_kernel(uint64_t* counters, uint64_t delay_ticks, uint64_t window_ticks) {
    const uint64_t arrival = __builtin_amdgcn_s_memrealtime();
    for (uint32_t i = 0; i < (1u << 24) && __builtin_amdgcn_s_memrealtime() - arrival < delay_ticks; ++i) __builtin_amdgcn_s_sleep(64);
    const uint64_t clock_begin = __builtin_amdgcn_s_memtime(), real_begin = __builtin_amdgcn_s_memrealtime();
    for (uint32_t i = 0; i < (1u << 24) && __builtin_amdgcn_s_memrealtime() - real_begin < window_ticks; ++i) __builtin_amdgcn_s_sleep(64);
    const uint64_t clock_end = __builtin_amdgcn_s_memtime(), real_end = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
        counters[0] = clock_end - clock_begin;
        counters[1] = real_end - real_begin;
    }
}

}  // namespace

// Enqueues the clock probe on `stream`: counters[0] / counters[1] x 100 MHz is the shader clock over the window.
extern "C" int bench_clock_probe(uint64_t* counters, uint64_t counter_bytes, uint64_t delay_ticks, uint64_t window_ticks, void* stream) {
    if (counters == nullptr || counter_bytes < 16 || window_ticks == 0 || delay_ticks + window_ticks > 100000000ull) return 1;
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), counters, delay_ticks, window_ticks);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

// Bytes of `operands` (2 * kOperandSets bf16x8 per thread), `sink` (one float per thread of the grid) and `counters`.
extern "C" uint64_t bench_mfma_sustained_operand_bytes(void) { return (uint64_t)2 * kOperandSets * kThreads * 16; }
extern "C" uint64_t bench_mfma_sustained_sink_bytes(uint32_t compute_units) { return (uint64_t)compute_units * kThreads * 4; }
extern "C" double bench_mfma_sustained_flops(uint32_t compute_units, uint32_t steps) {
    return (double)compute_units * (kThreads / 64) * (double)steps * kFlopsPerStep;
}

// Enqueues one launch on `stream` (never synchronized).  Returns 0, 1 for a bad argument, 2 for a HIP error.
extern "C" int bench_mfma_sustained(uint32_t tile32, const void* operands, uint64_t operand_bytes, float* sink, uint64_t sink_bytes,
                                    uint64_t* counters, uint64_t counter_bytes, uint32_t compute_units, uint32_t steps, void* stream) {
    if (operands == nullptr || sink == nullptr || counters == nullptr || compute_units == 0 || steps == 0) return 1;
    if (operand_bytes < bench_mfma_sustained_operand_bytes() || sink_bytes < bench_mfma_sustained_sink_bytes(compute_units) || counter_bytes < 16)
        return 1;
    const auto kernel = tile32 ? mfma_sustained_kernel<true> : mfma_sustained_kernel<false>;
    hipLaunchKernelGGL(kernel, dim3(compute_units), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(operands), sink, counters, steps);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
