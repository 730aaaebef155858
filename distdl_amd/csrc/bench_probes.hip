// Measurement aids of the benchmark (no counterpart in the reference, and not
// part of libdistdl_hip or its header): kernels that isolate one cost so that
// the figures the product's kernels are judged against -- what a launch costs
// by itself, what the matrix cores sustain on a given kind of data -- are
// measured on the same machine, in the same way, as those kernels.  Built as
// libdistdl_bench_probes.so, which only bench.py loads.
//
//   int bench_probe_launch(int64_t workgroups, int threads, void* stream)
//       enqueues a kernel that does nothing: the floor under every small kernel
//   int bench_probe_mfma(int instruction, int random, int iters, float* sink,
//                        int64_t sink_elems, int64_t* flop, void* stream)
//       enqueues a kernel of nothing but bf16 MFMAs on register operands (512
//       workgroups of 256 threads: two wavefronts per SIMD on 256 CUs);
//       instruction 0: v_mfma_f32_32x32x16_bf16, 1: v_mfma_f32_16x16x32_bf16;
//       random 0: every operand element 1.0, 1: N(0,1) x 0.02 N(0,1) operands
//       (on random operands the chip runs against its power limit); `iters`
//       loop iterations of 2^20 flop per wavefront, the flop count of the launch
//       is stored to the host address `flop` (may be NULL); `sink`: device
//       memory for 131072 floats that the kernel overwrites.
// Both return 0, -2 for a bad argument, or the hipError_t of the launch.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ddl {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__global__ void probe_kernel() {}

__device__ inline uint32_t mix(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// N(0,1) from two hashed uniforms (Box-Muller); only the statistics matter.
__device__ inline float gauss(uint32_t seed) {
    const float u1 = (mix(seed) >> 8) * (1.0f / 16777216.0f) + 1e-7f, u2 = (mix(seed ^ 0x9e3779b9U) >> 8) * (1.0f / 16777216.0f);
    return sqrtf(-2.f * logf(u1)) * cosf(6.2831853f * u2);
}

__device__ inline bf16x8 operand(uint32_t seed, float scale, int random) {
    bf16x8 v;
    for (int i = 0; i < 8; ++i) v[i] = static_cast<__bf16>(random ? scale * gauss(seed * 8 + i) : 1.0f);
    return v;
}

constexpr int kProbeBlocks = 512, kProbeThreads = 256;   // two wavefronts per SIMD on 256 CUs
constexpr int64_t kProbeFlopPerWaveIter = 1048576;        // both kernels: 2^20 flop per wavefront and iteration

// Nothing but MFMAs on operands that stay in registers: TN x TM accumulator
// tiles, two operand sets, the loop order of the shard GEMM's k-step.  32 MFMAs
// of 32x32x16 (8 tiles x 2 sets x 2) or 64 of 16x16x32 (32 tiles x 2 sets) per
// iteration.
__global__ __launch_bounds__(kProbeThreads) void mfma_probe_32x32x16(float* sink, int iters, int random) {
    constexpr int TN = 2, TM = 4;
    const uint32_t t = blockIdx.x * kProbeThreads + threadIdx.x;
    bf16x8 a[TN][2], b[TM][2];
    for (int i = 0; i < TN; ++i)
        for (int s = 0; s < 2; ++s) a[i][s] = operand(t * 64 + i * 2 + s, 0.02f, random);
    for (int i = 0; i < TM; ++i)
        for (int s = 0; s < 2; ++s) b[i][s] = operand(t * 64 + 32 + i * 2 + s, 1.0f, random);
    floatx16 acc[TN][TM];
    for (int i = 0; i < TN; ++i)
        for (int j = 0; j < TM; ++j)
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < 2 * iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
    }
    float sum = 0.f;
    for (int i = 0; i < TN; ++i)
        for (int j = 0; j < TM; ++j)
            for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
    sink[t] = sum;
}

__global__ __launch_bounds__(kProbeThreads) void mfma_probe_16x16x32(float* sink, int iters, int random) {
    constexpr int TN = 4, TM = 8;
    const uint32_t t = blockIdx.x * kProbeThreads + threadIdx.x;
    bf16x8 a[TN][2], b[TM][2];
    for (int i = 0; i < TN; ++i)
        for (int s = 0; s < 2; ++s) a[i][s] = operand(t * 64 + i * 2 + s, 0.02f, random);
    for (int i = 0; i < TM; ++i)
        for (int s = 0; s < 2; ++s) b[i][s] = operand(t * 64 + 32 + i * 2 + s, 1.0f, random);
    floatx4 acc[TN][TM];
    for (int i = 0; i < TN; ++i)
        for (int j = 0; j < TM; ++j)
            for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
    }
    float sum = 0.f;
    for (int i = 0; i < TN; ++i)
        for (int j = 0; j < TM; ++j)
            for (int e = 0; e < 4; ++e) sum += acc[i][j][e];
    sink[t] = sum;
}

}  // namespace
}  // namespace ddl

extern "C" {

int bench_probe_launch(int64_t workgroups, int threads, void* stream) {
    if (workgroups < 1 || workgroups > 0x7FFFFFFFll || threads < 1 || threads > 1024) return -2;
    hipLaunchKernelGGL(ddl::probe_kernel, dim3(static_cast<uint32_t>(workgroups)), dim3(threads), 0, static_cast<hipStream_t>(stream));
    return static_cast<int>(hipGetLastError());
}

int bench_probe_mfma(int instruction, int random, int iters, float* sink, int64_t sink_elems, int64_t* flop, void* stream) {
    using namespace ddl;
    if ((instruction != 0 && instruction != 1) || iters < 1 || iters > (1 << 24)) return -2;
    if (!sink || sink_elems < static_cast<int64_t>(kProbeBlocks) * kProbeThreads) return -2;
    if (flop) *flop = static_cast<int64_t>(kProbeBlocks) * (kProbeThreads / 64) * iters * kProbeFlopPerWaveIter;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (instruction == 0)
        hipLaunchKernelGGL(mfma_probe_32x32x16, dim3(kProbeBlocks), dim3(kProbeThreads), 0, s, sink, iters, random ? 1 : 0);
    else
        hipLaunchKernelGGL(mfma_probe_16x16x32, dim3(kProbeBlocks), dim3(kProbeThreads), 0, s, sink, iters, random ? 1 : 0);
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
