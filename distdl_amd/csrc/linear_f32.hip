// DistributedLinear shard in fp32: y[M,N] = a[M,K] . b[N,K]^T + bias[N] with
// fp32 operands, fp32 accumulation on the matrix cores (v_mfma_f32_32x32x2_f32)
// and an fp32 result (reference: nn/linear.py:103, nn/linear_ag.py:486 --
// torch.nn.functional.linear on the layer's default dtype, which is what the
// reference's own layer tests run, tests/layers/test_linear.py:48-305).
//
// Both operands are addressed by a row stride and a stride along the reduction
// dimension, so the products of the backward pass (dx = dy . w, dw = dy^T . x),
// whose operands are not contiguous along the reduction, need no transposed
// copies: a tile is fetched along whichever of its two dimensions is contiguous
// in memory.
//
//   workgroup  256 threads = 4 wavefronts (2 x 2), tile 128(m) x 128(n) x 16(k)
//   wavefront  64 x 64 = 2 x 2 tiles of 32 x 32, 64 accumulators per lane; the
//              product is formed transposed (b rows feed the A port, a rows the B
//              port) so a lane holds four consecutive n of one output row
//   LDS        two stages of (a tile + b tile), rows of 16 floats padded to 17
//              so that the 32 rows a fragment read touches fall on 32 banks
//   global     a thread fetches eight elements of each tile per k-tile into
//              registers (the next tile's, while the current one is multiplied)
//              and stores them to the other stage
//
// This kernel takes any strides, alignment and size; products large enough to
// fill the chip with 256 x 256 tiles whose operands have a unit stride and
// 16-byte alignment go to the tiled kernel of linear_f32_tiles.hip instead.
#include "ddl_common.h"

namespace ddl {

bool gemm_f32_tiled(const float* a, int64_t a_rs, int64_t a_ks, const float* b, int64_t b_rs, int64_t b_ks, const float* bias, float* y,
                    int64_t ldy, int64_t M, int64_t N, int64_t K, void* stream, int* rc);

namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

constexpr int kThreads = 256;
constexpr int BM = 128, BN = 128, BK = 16;
constexpr int kPitch = BK + 1;                 // floats per LDS row
constexpr int kTileFloats = 128 * kPitch;      // one operand tile in LDS
constexpr int kPerThread = 128 * BK / kThreads;   // elements of a tile a thread fetches: 8

struct Operand {
    const float* p;    // first row of the workgroup's tile is p + row0 * rs
    int64_t rs, ks;    // element strides between rows and along the reduction
    int64_t rows;      // rows of the matrix (M or N)
};

// How a thread's eight elements of a 128 x 16 tile are laid out.
//   ALONG_K: the reduction is contiguous in memory: thread t takes row t / 2,
//            reduction elements 8 (t % 2) .. + 7 (two 16-byte loads when aligned)
//   else     rows are contiguous (or nothing is): thread t takes reduction
//            element t / 16 and rows 8 (t % 16) .. + 7, so that neighbouring
//            threads read neighbouring rows
template <bool ALONG_K>
__device__ inline void fetch(const Operand& o, int64_t row0, int64_t k0, int64_t K, bool vec, float (&v)[kPerThread]) {
    const int t = threadIdx.x;
    if (ALONG_K) {
        const int64_t r = row0 + (t >> 1), k = k0 + 8 * (t & 1);
        const bool row_ok = r < o.rows;
        const float* src = o.p + r * o.rs + k * o.ks;
        if (vec && row_ok && k + 8 <= K) {
            const float4 q0 = *reinterpret_cast<const float4*>(src), q1 = *reinterpret_cast<const float4*>(src + 4);
            v[0] = q0.x, v[1] = q0.y, v[2] = q0.z, v[3] = q0.w, v[4] = q1.x, v[5] = q1.y, v[6] = q1.z, v[7] = q1.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (row_ok && k + e < K) ? src[e * o.ks] : 0.f;
        }
    } else {
        const int64_t k = k0 + (t >> 4), r = row0 + 8 * (t & 15);
        const bool k_ok = k < K;
        const float* src = o.p + r * o.rs + k * o.ks;
        if (vec && k_ok && r + 8 <= o.rows) {
            const float4 q0 = *reinterpret_cast<const float4*>(src), q1 = *reinterpret_cast<const float4*>(src + 4);
            v[0] = q0.x, v[1] = q0.y, v[2] = q0.z, v[3] = q0.w, v[4] = q1.x, v[5] = q1.y, v[6] = q1.z, v[7] = q1.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (k_ok && r + e < o.rows) ? src[e * o.rs] : 0.f;
        }
    }
}

template <bool ALONG_K>
__device__ inline void stash(float* tile, const float (&v)[kPerThread]) {
    const int t = threadIdx.x;
    if (ALONG_K) {
        float* dst = tile + (t >> 1) * kPitch + 8 * (t & 1);
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e] = v[e];
    } else {
        float* dst = tile + 8 * (t & 15) * kPitch + (t >> 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e * kPitch] = v[e];
    }
}

template <bool A_ALONG_K, bool B_ALONG_K>
__global__ __launch_bounds__(kThreads) void gemm_f32_kernel(const Operand a, const Operand b, const float* __restrict__ bias,
                                                            float* __restrict__ y, int64_t ldy, int64_t K, int tiles_m,
                                                            int a_vec, int b_vec) {
    __shared__ float lds[2][2][kTileFloats];   // [stage][a / b]
    // XCD-aware tile assignment: hardware deals workgroup ids round-robin over
    // the 8 XCDs, so id % 8 names the XCD.  Each XCD gets a contiguous range of
    // the tile sequence, which is walked in bands of 8 m-tiles, so that the
    // workgroups resident on an XCD share operand panels in its L2.
    const int ntiles = gridDim.x;
    const int tiles_n = ntiles / tiles_m;
    int id = blockIdx.x;
    {
        const int per = ntiles / 8, main = per * 8;
        if (id < main) id = (id % 8) * per + id / 8;
    }
    constexpr int kBand = 8;
    const int band = id / (kBand * tiles_n);
    const int band_m0 = band * kBand;
    const int band_h = (tiles_m - band_m0) < kBand ? (tiles_m - band_m0) : kBand;
    const int in_band = id - band * kBand * tiles_n;
    const int tm = band_m0 + in_band % band_h, tn = in_band / band_h;
    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = (wave & 1) * 64, wn = (wave >> 1) * 64;
    const int l32 = lane & 31, kg = lane >> 5;

    floatx16 acc[2][2];   // [n sub-tile][m sub-tile]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int64_t ktiles = (K + BK - 1) / BK;
    float va[kPerThread], vb[kPerThread];
    fetch<A_ALONG_K>(a, m0, 0, K, a_vec, va);
    fetch<B_ALONG_K>(b, n0, 0, K, b_vec, vb);
    stash<A_ALONG_K>(lds[0][0], va);
    stash<B_ALONG_K>(lds[0][1], vb);
    __syncthreads();
    for (int64_t t = 0; t < ktiles; ++t) {
        const int cur = static_cast<int>(t & 1);
        if (t + 1 < ktiles) {
            fetch<A_ALONG_K>(a, m0, (t + 1) * BK, K, a_vec, va);
            fetch<B_ALONG_K>(b, n0, (t + 1) * BK, K, b_vec, vb);
        }
        const float* ta = lds[cur][0];
        const float* tb = lds[cur][1];
#pragma unroll
        for (int kk = 0; kk < BK / 2; ++kk) {
            float fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fb[i] = tb[(wn + 32 * i + l32) * kPitch + 2 * kk + kg];   // b rows -> A port
                fa[i] = ta[(wm + 32 * i + l32) * kPitch + 2 * kk + kg];   // a rows -> B port
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[i], fa[j], acc[i][j], 0, 0, 0);
        }
        if (t + 1 < ktiles) {
            // the other stage was last read in iteration t - 1, which every wavefront left through the barrier below
            stash<A_ALONG_K>(lds[cur ^ 1][0], va);
            stash<B_ALONG_K>(lds[cur ^ 1][1], vb);
        }
        __syncthreads();
    }
    // Lane holds, per 32 x 32 tile, output row m = l32 and columns n = 8 g + 4 kg + {0..3} in acc[..][4 g + {0..3}].
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int64_t n = n0 + wn + 32 * i + 8 * g + 4 * kg;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < b.rows) bv[e] = bias[n + e];
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int64_t m = m0 + wm + 32 * j + l32;
                if (m >= a.rows) continue;
                float* dst = y + m * ldy + n;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < b.rows) dst[e] = acc[i][j][4 * g + e] + bv[e];
            }
        }
    }
}

// An operand can be fetched 16 bytes at a time along its contiguous dimension
// when base and the other stride keep every such piece aligned.
bool vector_ok(const Operand& o, bool along_k) {
    const int64_t other = along_k ? o.rs : o.ks;
    return aligned_to(o.p, 16) && other % 4 == 0;
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_gemm_f32(const float* a, int64_t a_row_stride, int64_t a_k_stride, const float* b, int64_t b_row_stride,
                            int64_t b_k_stride, const float* bias, float* y, int64_t ldy, int64_t M, int64_t N, int64_t K,
                            void* stream) {
    using namespace ddl;
    if (M < 0 || N < 0 || K < 0 || ldy < N)
        return fail(DDL_E_ARG, "gemm f32: M=%lld N=%lld K=%lld ldy=%lld", (long long)M, (long long)N, (long long)K, (long long)ldy);
    if (M == 0 || N == 0) return 0;
    if (!a || !b || !y) return fail(DDL_E_ARG, "gemm f32: null pointer");
    if (K == 0) return fail(DDL_E_UNSUPP, "gemm f32: K = 0");
    if (a_row_stride < 0 || a_k_stride < 0 || b_row_stride < 0 || b_k_stride < 0) return fail(DDL_E_ARG, "gemm f32: negative stride");
    if (!aligned_to(a, 4) || !aligned_to(b, 4) || !aligned_to(y, 4) || !aligned_to(bias, 4)) return fail(DDL_E_ALIGN, "gemm f32: pointer misaligned");
    // At least a quarter of the CUs' worth of 256 x 256 tiles: below that, the 128 x 128 tiles here spread the work further.
    if (((M + 255) / 256) * ((N + 255) / 256) >= 64) {
        int rc = 0;
        if (gemm_f32_tiled(a, a_row_stride, a_k_stride, b, b_row_stride, b_k_stride, bias, y, ldy, M, N, K, stream, &rc)) return rc;
    }
    const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7FFFFFFFll || tiles_m > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "gemm f32: too many output tiles");
    const Operand oa{a, a_row_stride, a_k_stride, M}, ob{b, b_row_stride, b_k_stride, N};
    const bool a_k = a_k_stride == 1 || a_row_stride != 1, b_k = b_k_stride == 1 || b_row_stride != 1;
    const int a_vec = (a_k ? a_k_stride == 1 : a_row_stride == 1) && vector_ok(oa, a_k) ? 1 : 0;
    const int b_vec = (b_k ? b_k_stride == 1 : b_row_stride == 1) && vector_ok(ob, b_k) ? 1 : 0;
    const dim3 grid(static_cast<uint32_t>(tiles_m * tiles_n));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int tm = static_cast<int>(tiles_m);
    if (a_k && b_k)
        hipLaunchKernelGGL((gemm_f32_kernel<true, true>), grid, dim3(kThreads), 0, s, oa, ob, bias, y, ldy, K, tm, a_vec, b_vec);
    else if (a_k)
        hipLaunchKernelGGL((gemm_f32_kernel<true, false>), grid, dim3(kThreads), 0, s, oa, ob, bias, y, ldy, K, tm, a_vec, b_vec);
    else if (b_k)
        hipLaunchKernelGGL((gemm_f32_kernel<false, true>), grid, dim3(kThreads), 0, s, oa, ob, bias, y, ldy, K, tm, a_vec, b_vec);
    else
        hipLaunchKernelGGL((gemm_f32_kernel<false, false>), grid, dim3(kThreads), 0, s, oa, ob, bias, y, ldy, K, tm, a_vec, b_vec);
    return check_launch("gemm_f32_kernel");
}
