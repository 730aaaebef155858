// DistributedLinear shard GEMM: y[M,N] = x[M,K] . w[N,K]^T + bias[N], bf16
// operands, fp32 accumulation on the matrix cores, bf16 result (reference:
// nn/linear.py:103, nn/linear_ag.py:486 -- torch.nn.functional.linear).
//
// Both operands are K-contiguous, so a 16-byte load anywhere gives eight
// consecutive k of one row: exactly one lane's share of an MFMA operand.  The
// product is formed transposed (w rows feed the A port, x rows the B port) so
// that each lane ends up with four consecutive n of one output row and can
// store them as one 8-byte word.
//
//   workgroup  512 threads = 8 wavefronts (2 along m x 4 along n), tile
//              256(m) x 256(n) x 64(k); two wavefronts share a SIMD so that one
//              can issue MFMAs while the other waits for LDS
//   wavefront  128(m) x 64(n) = 4 x 2 tiles of v_mfma_f32_32x32x16_bf16, 128 fp32
//              accumulators per lane
//   LDS        two stages of {w tile, x tile} = 2 x 64 KiB; rows are 128 B with
//              the 16-byte chunk index XOR-ed by ((row >> 1) & 7): the 16 lanes
//              served per LDS cycle read 16 consecutive rows, and (row & 1,
//              (row >> 1) & 7) is distinct for each, so they cover all 64 banks
//   schedule   global loads of k-tile t+1 are issued before the MFMAs of tile
//              t and written to the other LDS stage after them; one barrier
//              per k-tile
//   launch     workgroup ids are regrouped so that the 32 workgroups resident
//              on one XCD cover a compact patch of the tile grid and share
//              their operand panels in that XCD's L2
#include "ddl_common.h"

namespace ddl {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 512;
constexpr int kTileBytes = BM * BK * 2;          // one operand tile, 32 KiB
constexpr int kStageBytes = 2 * kTileBytes;      // w tile + x tile
constexpr int kLdsBytes = 2 * kStageBytes;       // two stages
constexpr int kXcds = 8;

__device__ inline uint32_t lds_offset(int row, int chunk) { return row * (BK * 2) + ((chunk ^ ((row >> 1) & 7)) << 4); }

__device__ inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7FC0;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ inline float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// Loads this thread's four 16-byte chunks of one operand tile (rows row0..+255
// of a [rows_total, K] matrix, columns k0..k0+63).  Rows past the end repeat the
// last valid row (their products are never stored); chunks past K read as zero.
__device__ inline void load_tile(const uint16_t* __restrict__ g, int64_t ld, int64_t rows_total, int64_t row0, int64_t K,
                                 int64_t k0, uint4 (&r)[4]) {
    const int c = threadIdx.x & 7;
    const int rr = threadIdx.x >> 3;
    const int64_t k = k0 + c * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int64_t row = row0 + rr + 64 * i;
        row = row < rows_total ? row : rows_total - 1;
        if (k < K)
            r[i] = *reinterpret_cast<const uint4*>(g + row * ld + k);
        else
            r[i] = make_uint4(0, 0, 0, 0);
    }
}

__device__ inline void store_tile(char* lds, const uint4 (&r)[4]) {
    const int c = threadIdx.x & 7;
    const int rr = threadIdx.x >> 3;
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(lds + lds_offset(rr + 64 * i, c)) = r[i];
}

__global__ __launch_bounds__(kThreads) void linear_bf16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                               const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
                                                               int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw,
                                                               int64_t ldy, int tiles_m, int tiles_n, int vec_store) {
    extern __shared__ __attribute__((aligned(16))) char lds[];

    // XCD-aware tile assignment: hardware deals workgroup ids round-robin over
    // the XCDs, so id % 8 names the XCD.  Give each XCD a contiguous range of
    // the tile sequence, and walk that sequence in bands of 8 m-tiles.
    const int ntiles = tiles_m * tiles_n;
    int id = blockIdx.x;
    {
        const int per = ntiles / kXcds, main = per * kXcds;
        if (id < main) id = (id % kXcds) * per + id / kXcds;
    }
    constexpr int kBand = 8;
    const int band = id / (kBand * tiles_n);
    const int band_m0 = band * kBand;
    const int band_h = (tiles_m - band_m0) < kBand ? (tiles_m - band_m0) : kBand;
    const int in_band = id - band * kBand * tiles_n;
    const int tm = band_m0 + in_band % band_h;
    const int tn = in_band / band_h;

    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = (wave & 1) * 128, wn = (wave >> 1) * 64;   // wavefront origin inside the tile
    const int l32 = lane & 31, kg = lane >> 5;

    constexpr int TN = 2, TM = 4;   // 32x32 sub-tiles of a wavefront along n and m
    floatx16 acc[TN][TM];  // [n sub-tile][m sub-tile]
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    uint4 rw[4], rx[4];
    const int64_t ktiles = (K + BK - 1) / BK;
    load_tile(w, ldw, N, n0, K, 0, rw);
    load_tile(x, ldx, M, m0, K, 0, rx);
    store_tile(lds, rw);
    store_tile(lds + kTileBytes, rx);
    __syncthreads();

    for (int64_t kt = 0; kt < ktiles; ++kt) {
        char* cur = lds + (kt & 1) * kStageBytes;
        char* nxt = lds + ((kt + 1) & 1) * kStageBytes;
        const bool more = kt + 1 < ktiles;
        if (more) {
            load_tile(w, ldw, N, n0, K, (kt + 1) * BK, rw);
            load_tile(x, ldx, M, m0, K, (kt + 1) * BK, rx);
        }
        const char* sw = cur;
        const char* sx = cur + kTileBytes;
        // Operand fragments are double-buffered: the LDS reads of k-step ks+1
        // are issued before the MFMAs of k-step ks, so a wavefront does not
        // stall on LDS latency between k-steps.
        bf16x8 fa[2][TN], fb[2][TM];
#pragma unroll
        for (int a = 0; a < TN; ++a) fa[0][a] = *reinterpret_cast<const bf16x8*>(sw + lds_offset(wn + a * 32 + l32, kg));
#pragma unroll
        for (int b = 0; b < TM; ++b) fb[0][b] = *reinterpret_cast<const bf16x8*>(sx + lds_offset(wm + b * 32 + l32, kg));
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const int cb = ks & 1, nb = cb ^ 1;
            const bool pre = ks + 1 < BK / 16;
            // One LDS read of the next k-step is issued behind each MFMA of this
            // one, so that LDS traffic is spread evenly instead of arriving in
            // bursts that fill the LDS queues of all wavefronts at once.
#pragma unroll
            for (int i = 0; i < TN * TM; ++i) {
                const int a = i / TM, b = i % TM;
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cb][a], fb[cb][b], acc[a][b], 0, 0, 0);
                if (pre && i < TN)
                    fa[nb][i] = *reinterpret_cast<const bf16x8*>(sw + lds_offset(wn + i * 32 + l32, (ks + 1) * 2 + kg));
                else if (pre && i < TN + TM)
                    fb[nb][i - TN] = *reinterpret_cast<const bf16x8*>(sx + lds_offset(wm + (i - TN) * 32 + l32, (ks + 1) * 2 + kg));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (more) {
            store_tile(nxt, rw);
            store_tile(nxt + kTileBytes, rx);
        }
        __syncthreads();
    }

    // Epilogue.  Lane holds, per 32x32 tile, output row m = l32 and the columns
    // n = 8*g + 4*kg + {0,1,2,3} for g = 0..3 in acc[...][4*g + {0..3}].
#pragma unroll
    for (int a = 0; a < TN; ++a) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int64_t n = n0 + wn + a * 32 + 8 * g + 4 * kg;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) bv[e] = bf16_bits_to_f32(bias[n + e]);
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int64_t m = m0 + wm + b * 32 + l32;
                if (m >= M) continue;
                uint16_t o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16_bits(acc[a][b][4 * g + e] + bv[e]);
                uint16_t* dst = y + m * ldy + n;
                if (vec_store && n + 3 < N) {
                    uint2 pk;
                    pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
                    pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
                    *reinterpret_cast<uint2*>(dst) = pk;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) dst[e] = o[e];
                }
            }
        }
    }
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_linear_bf16(const void* x, const void* w, const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                               int64_t ldx, int64_t ldw, int64_t ldy, void* stream) {
    using namespace ddl;
    if (M < 0 || N < 0 || K < 0 || ldx < K || ldw < K || ldy < N)
        return fail(DDL_E_ARG, "linear: M=%lld N=%lld K=%lld ldx=%lld ldw=%lld ldy=%lld", (long long)M, (long long)N,
                    (long long)K, (long long)ldx, (long long)ldw, (long long)ldy);
    if (M == 0 || N == 0) return 0;
    if (!x || !w || !y) return fail(DDL_E_ARG, "linear: null pointer");
    if (K == 0) return fail(DDL_E_UNSUPP, "linear: K = 0");
    if (K % 8 != 0 || ldx % 8 != 0 || ldw % 8 != 0 || !aligned_to(x, 16) || !aligned_to(w, 16))
        return fail(DDL_E_ALIGN, "linear: K, ldx, ldw must be multiples of 8 and x, w 16-byte aligned");
    if (!aligned_to(y, 2) || (bias && !aligned_to(bias, 2))) return fail(DDL_E_ALIGN, "linear: y / bias misaligned");
    const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7FFFFFFFll || tiles_m > 0x7FFFFFll || tiles_n > 0x7FFFFFll)
        return fail(DDL_E_UNSUPP, "linear: too many output tiles");
    static bool attr_done = false;
    if (!attr_done) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(linear_bf16_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e != hipSuccess) return fail(static_cast<int>(e), "linear: cannot reserve %d bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
        attr_done = true;
    }
    const int vec_store = (ldy % 4 == 0) && aligned_to(y, 8);
    hipLaunchKernelGGL(linear_bf16_kernel, dim3(static_cast<uint32_t>(tiles_m * tiles_n)), dim3(kThreads), kLdsBytes,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w),
                       static_cast<const uint16_t*>(bias), static_cast<uint16_t*>(y), M, N, K, ldx, ldw, ldy,
                       static_cast<int>(tiles_m), static_cast<int>(tiles_n), vec_store);
    return check_launch("linear_bf16_kernel");
}
