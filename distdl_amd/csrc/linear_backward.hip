// Helpers of the DistributedLinear shard backward (the adjoint of
// torch.nn.functional.linear, reference: nn/linear.py:103, nn/linear_ag.py:486):
//
//   dx[M,K] = dy[M,N] . w[N,K]          reduction over N
//   dw[N,K] = dy[M,N]^T . x[M,K]        reduction over M
//   db[N]   = sum over m of dy[m,N]
//
// The shard GEMM multiplies two operands that are contiguous along the
// reduction dimension.  dy is (for dx); w, dy and x (for dx and dw) are not, so
// they are transposed once into a workspace -- a pass over 2 bytes per element
// each way, small next to the GEMM -- and the same GEMM kernel does the rest.
// db is a column sum with fp32 accumulation.
#include "ddl_common.h"

#include <hip/hip_fp16.h>

namespace ddl {
namespace {

constexpr int kTile = 64;      // elements per tile edge
constexpr int kBlock = 256;

// dst[c, r] = src[r, c] for 16-bit elements.  A 64 x 64 tile goes through LDS:
// rows are read 16 bytes per lane, the transposed rows are put together from
// 2-byte LDS reads and written 16 bytes per lane.  The LDS row pitch of 66
// elements (33 dwords) spreads a column over all banks.
__global__ __launch_bounds__(kBlock) void transpose16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                             int64_t rows, int64_t cols, int64_t ld_src, int64_t ld_dst,
                                                             int tiles_c, int vec_ok) {
    __shared__ uint16_t tile[kTile][kTile + 2];
    const int tr = blockIdx.x / tiles_c, tc = blockIdx.x - tr * tiles_c;
    const int64_t r0 = static_cast<int64_t>(tr) * kTile, c0 = static_cast<int64_t>(tc) * kTile;
    const int t = threadIdx.x;
    // load: 8 lanes per row (8 x 8 elements), 32 rows per pass
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int r = (t >> 3) + 32 * p, c = (t & 7) * 8;
        const int64_t gr = r0 + r, gc = c0 + c;
        uint16_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (gr < rows) {
            const uint16_t* s = src + gr * ld_src + gc;
            if (vec_ok && gc + 8 <= cols) {
                const uint4 q = *reinterpret_cast<const uint4*>(s);
                v[0] = q.x & 0xFFFF; v[1] = q.x >> 16; v[2] = q.y & 0xFFFF; v[3] = q.y >> 16;
                v[4] = q.z & 0xFFFF; v[5] = q.z >> 16; v[6] = q.w & 0xFFFF; v[7] = q.w >> 16;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (gc + e < cols) v[e] = s[e];
            }
        }
#pragma unroll
        for (int e = 0; e < 8; e += 2)
            *reinterpret_cast<uint32_t*>(&tile[r][c + e]) = static_cast<uint32_t>(v[e]) | (static_cast<uint32_t>(v[e + 1]) << 16);
    }
    __syncthreads();
    // store: output row = source column; 8 lanes per output row, 8 source rows each
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int oc = (t >> 3) + 32 * p, orr = (t & 7) * 8;   // source column, first source row
        const int64_t gc = c0 + oc, gr = r0 + orr;
        if (gc >= cols || gr >= rows) continue;
        uint16_t v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = tile[orr + e][oc];
        uint16_t* d = dst + gc * ld_dst + gr;
        if (vec_ok && gr + 8 <= rows) {
            uint4 q;
            q.x = v[0] | (static_cast<uint32_t>(v[1]) << 16);
            q.y = v[2] | (static_cast<uint32_t>(v[3]) << 16);
            q.z = v[4] | (static_cast<uint32_t>(v[5]) << 16);
            q.w = v[6] | (static_cast<uint32_t>(v[7]) << 16);
            *reinterpret_cast<uint4*>(d) = q;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (gr + e < rows) d[e] = v[e];
        }
    }
}

__device__ inline float bf16_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

__device__ inline uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7FC0;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// Element types of the column sum: 0 = bf16, 1 = fp16, 2 = fp32.
template <int DT>
struct Elem;
template <>
struct Elem<0> {
    typedef uint16_t type;
    static __device__ float load(const uint16_t* p) { return bf16_to_f32(*p); }
    static __device__ void store(uint16_t* p, float f) { *p = f32_to_bf16(f); }
    static __device__ void load8(const uint16_t* p, float (&v)[8]) {
        const uint4 q = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[2 * e] = __uint_as_float(w[e] << 16);
            v[2 * e + 1] = __uint_as_float(w[e] & 0xFFFF0000u);
        }
    }
};
template <>
struct Elem<1> {
    typedef __half type;
    static __device__ float load(const __half* p) { return __half2float(*p); }
    static __device__ void store(__half* p, float f) { *p = __float2half_rn(f); }
    static __device__ void load8(const __half* p, float (&v)[8]) {
        const uint4 q = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float2 f = __half22float2(*reinterpret_cast<const __half2*>(&w[e]));
            v[2 * e] = f.x;
            v[2 * e + 1] = f.y;
        }
    }
};
template <>
struct Elem<2> {
    typedef float type;
    static __device__ float load(const float* p) { return *p; }
    static __device__ void store(float* p, float f) { *p = f; }
    static __device__ void load8(const float* p, float (&v)[8]) {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    }
};

// Stage 1 of the column sum: workgroup (strip, split) adds rows
// [split * rows_per_split, ...) of a 64-column strip in fp32 and writes 64
// partial sums to partial[split, col].  8 lanes cover the 64 columns of a row,
// 32 rows are in flight per pass; LDS folds the 32 row groups.
template <int DT>
__global__ __launch_bounds__(kBlock) void colsum_partial_kernel(const typename Elem<DT>::type* __restrict__ a, int64_t rows, int64_t cols,
                                                                int64_t ld, int64_t rows_per_split, float* __restrict__ partial,
                                                                int strips, int vec_ok) {
    __shared__ float fold[32][kTile + 1];
    const int split = blockIdx.x / strips, strip = blockIdx.x - split * strips;
    const int t = threadIdx.x;
    const int g = t >> 3, c = (t & 7) * 8;
    const int64_t gc = static_cast<int64_t>(strip) * kTile + c;
    const int64_t r_begin = split * rows_per_split;
    const int64_t r_end = r_begin + rows_per_split < rows ? r_begin + rows_per_split : rows;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (vec_ok && gc + 8 <= cols) {
        for (int64_t r = r_begin + g; r < r_end; r += 32) {
            float v[8];
            Elem<DT>::load8(a + r * ld + gc, v);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += v[e];
        }
    } else {
        for (int64_t r = r_begin + g; r < r_end; r += 32) {
            const typename Elem<DT>::type* s = a + r * ld + gc;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (gc + e < cols) acc[e] += Elem<DT>::load(s + e);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) fold[g][c + e] = acc[e];
    __syncthreads();
    if (t < kTile) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 32; ++k) s += fold[k][t];
        const int64_t col = static_cast<int64_t>(strip) * kTile + t;
        if (col < cols) partial[static_cast<int64_t>(split) * cols + col] = s;
    }
}

// Stage 2: out[col] = sum over splits of partial[split, col], rounded to the element type.  A workgroup
// per 64-column strip; lane group t / 64 adds every fourth split (eight
// independent loads in flight), LDS folds the four groups.
template <int DT>
__global__ __launch_bounds__(kBlock) void colsum_final_kernel(const float* __restrict__ partial, int64_t cols, int splits,
                                                              typename Elem<DT>::type* __restrict__ out) {
    constexpr int kGroups = kBlock / kTile;
    __shared__ float fold[kGroups][kTile];
    const int g = threadIdx.x / kTile, t = threadIdx.x % kTile;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * kTile + t;
    float s = 0.f;
    if (col < cols) {
        int k = g;
        for (; k + 7 * kGroups < splits; k += 8 * kGroups) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[static_cast<int64_t>(k + u * kGroups) * cols + col];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; k < splits; k += kGroups) s += partial[static_cast<int64_t>(k) * cols + col];
    }
    fold[g][t] = s;
    __syncthreads();
    if (g == 0 && col < cols) {
        float r = 0.f;
#pragma unroll
        for (int k = 0; k < kGroups; ++k) r += fold[k][t];
        Elem<DT>::store(out + col, r);
    }
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_transpose_2d(const void* src, void* dst, int64_t rows, int64_t cols, int64_t ld_src, int64_t ld_dst,
                                int elem_size, void* stream) {
    using namespace ddl;
    if (rows < 0 || cols < 0 || ld_src < cols || ld_dst < rows)
        return fail(DDL_E_ARG, "transpose: rows=%lld cols=%lld ld_src=%lld ld_dst=%lld", (long long)rows, (long long)cols,
                    (long long)ld_src, (long long)ld_dst);
    if (elem_size != 2) return fail(DDL_E_UNSUPP, "transpose: element size %d (only 2-byte elements)", elem_size);
    if (rows == 0 || cols == 0) return 0;
    if (!src || !dst) return fail(DDL_E_ARG, "transpose: null pointer");
    if (!aligned_to(src, 2) || !aligned_to(dst, 2)) return fail(DDL_E_ALIGN, "transpose: pointer misaligned");
    const int64_t tiles_r = (rows + kTile - 1) / kTile, tiles_c = (cols + kTile - 1) / kTile;
    if (tiles_r * tiles_c > 0x7FFFFFFFll || tiles_c > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "transpose: too many tiles");
    const int vec_ok = aligned_to(src, 16) && aligned_to(dst, 16) && ld_src % 8 == 0 && ld_dst % 8 == 0;
    hipLaunchKernelGGL(transpose16_kernel, dim3(static_cast<uint32_t>(tiles_r * tiles_c)), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), rows,
                       cols, ld_src, ld_dst, static_cast<int>(tiles_c), vec_ok);
    return check_launch("transpose16_kernel");
}

namespace ddl {
namespace {

template <int DT>
int run_colsum(const void* a, int64_t rows, int64_t cols, int64_t ld, void* out, float* workspace, int64_t splits,
               int64_t rows_per_split, int64_t strips, hipStream_t s) {
    typedef typename Elem<DT>::type T;
    const int vec_ok = (aligned_to(a, 8 * sizeof(T)) && (ld * sizeof(T)) % 16 == 0) ? 1 : 0;
    hipLaunchKernelGGL((colsum_partial_kernel<DT>), dim3(static_cast<uint32_t>(strips * splits)), dim3(kBlock), 0, s,
                       static_cast<const T*>(a), rows, cols, ld, rows_per_split, workspace, static_cast<int>(strips), vec_ok);
    const int rc = check_launch("colsum_partial_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL((colsum_final_kernel<DT>), dim3(static_cast<uint32_t>(strips)), dim3(kBlock), 0, s, workspace, cols,
                       static_cast<int>(splits), static_cast<T*>(out));
    return check_launch("colsum_final_kernel");
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_colsum(const void* a, int dtype, int64_t rows, int64_t cols, int64_t ld, void* out, float* workspace,
                          int64_t workspace_elems, void* stream) {
    using namespace ddl;
    if (dtype != DDL_DT_BF16 && dtype != DDL_DT_F16 && dtype != DDL_DT_F32) return fail(DDL_E_UNSUPP, "colsum: dtype %d (bf16, f16 and f32 only)", dtype);
    if (rows < 0 || cols < 0 || ld < cols) return fail(DDL_E_ARG, "colsum: rows=%lld cols=%lld ld=%lld", (long long)rows, (long long)cols, (long long)ld);
    if (cols == 0) return 0;
    if (!out || !workspace || (rows > 0 && !a)) return fail(DDL_E_ARG, "colsum: null pointer");
    const int es = dtype == DDL_DT_F32 ? 4 : 2;
    if (!aligned_to(a, es) || !aligned_to(out, es) || !aligned_to(workspace, 4)) return fail(DDL_E_ALIGN, "colsum: pointer misaligned");
    // as many row splits as the workspace holds, up to 64 and to 128 rows per split
    int64_t splits = workspace_elems / cols;
    if (splits < 1) return fail(DDL_E_ARG, "colsum: workspace of %lld floats is smaller than one row of %lld", (long long)workspace_elems, (long long)cols);
    if (splits > 64) splits = 64;
    const int64_t by_rows = (rows + 127) / 128;
    if (splits > by_rows) splits = by_rows > 0 ? by_rows : 1;
    const int64_t rows_per_split = rows > 0 ? (rows + splits - 1) / splits : 1;
    const int64_t strips = (cols + kTile - 1) / kTile;
    if (strips * splits > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "colsum: too many workgroups");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == DDL_DT_BF16) return run_colsum<0>(a, rows, cols, ld, out, workspace, splits, rows_per_split, strips, s);
    if (dtype == DDL_DT_F16) return run_colsum<1>(a, rows, cols, ld, out, workspace, splits, rows_per_split, strips, s);
    return run_colsum<2>(a, rows, cols, ld, out, workspace, splits, rows_per_split, strips, s);
}

extern "C" int ddl_colsum_bf16(const void* a, int64_t rows, int64_t cols, int64_t ld, void* out, float* workspace,
                               int64_t workspace_elems, void* stream) {
    return ddl_colsum(a, DDL_DT_BF16, rows, cols, ld, out, workspace, workspace_elems, stream);
}
